"""Two mixers side by side on the same normed rows: each output is divided by its root mean square over the
model's width and multiplied by a weight of its own, and the two are joined with fixed coefficients
(a half each: their mean). The two mixers are any registered kinds; their cache needs follow each other."""
import torch

from ..cache import StateNeed
from ..kernels import ops
from ..weights import TensorNeed
from .base import Part
from .registry import build, register


class _CacheOfOne:
    """The cache as one of the two mixers sees it: the fixed-size states of the entry that are its own."""

    def __init__(self, cache, first, count):
        self.cache, self.first, self.count = cache, first, count

    def kv_view(self, entry):
        return self.cache.kv_view(entry)

    def state_views(self, entry):
        return self.cache.state_views(entry)[self.first:self.first + self.count]


def _needs_of(mixer):
    need = mixer.cache_need()
    if need is None:
        return ()
    return tuple(need) if isinstance(need, (tuple, list)) else (need,)


@register("mixer", "side_by_side")
class SideBySide(Part):
    stores_fresh_rows = True     # the joined rows are stored into rows that hold nothing yet (StepContext.adds_to)

    def __init__(self, hidden_size, left, right, eps, names, weights=(0.5, 0.5), shared=None):
        """left, right: PartSpecs of mixers. names: left_norm, right_norm -> the tensors of the two output norms.
        weights: what each normed output is multiplied by in the sum."""
        self.hidden_size, self.eps = int(hidden_size), float(eps)
        self.sides = (build("mixer", left, shared=shared), build("mixer", right, shared=shared))
        self.weights = (float(weights[0]), float(weights[1]))
        self.names = dict(names)
        self.norm_w = None
        counts = [sum(isinstance(n, StateNeed) for n in _needs_of(m)) for m in self.sides]
        self.states = ((0, counts[0]), (counts[0], counts[1]))         # (first, count) of each side's states
        all_needs = [n for m in self.sides for n in _needs_of(m)]
        if len(set(all_needs)) != len(all_needs):
            raise ValueError("mixers side by side must not have two equal cache needs")

    @property
    def graph_safe(self):
        return all(getattr(m, "graph_safe", False) for m in self.sides)

    def tensor_needs(self):
        needs = {self.names["left_norm"]: TensorNeed((self.hidden_size,), "scale"),
                 self.names["right_norm"]: TensorNeed((self.hidden_size,), "scale")}
        for m in self.sides:
            needs.update(m.tensor_needs())
        return needs

    def cache_need(self):
        needs = tuple(n for m in self.sides for n in _needs_of(m))
        return needs or None

    def load(self, tensors, rt):
        for m in self.sides:
            m.load(tensors, rt)
        self.norm_w = tuple(rt.weight(tensors[self.names[k]], matrix=False) for k in ("left_norm", "right_norm"))

    def forward(self, ctx, y, x):
        rt = ctx.rt
        target, cache = ctx.fresh_rows, ctx.cache
        rows = []
        for side, (mixer, (first, count)) in enumerate(zip(self.sides, self.states)):
            out = rt.buffer(f"side_{side}", tuple(x.shape), torch.float32)
            ctx.handed = ctx.norm_ahead = ctx.left = None
            if getattr(mixer, "stores_fresh_rows", False):
                ctx.fresh_rows = out
            else:
                ctx.fresh_rows = None
                ops.fill_u32(out, 0)
            ctx.cache = _CacheOfOne(cache, first, count)
            try:
                mixer.forward(ctx, y, out)
            finally:
                ctx.cache, ctx.fresh_rows = cache, target
            rows.append(out)
        ops.normed_pair(rows[0], self.norm_w[0], self.weights[0], rows[1], self.norm_w[1], self.weights[1], x, self.eps,
                        accumulate=ctx.adds_to(x))
