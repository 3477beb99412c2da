"""Norms of the residual stream. RMSNorm as the reference computes it (crates/backends/backend_common/src/kernels.rs:54-64):
y = x / sqrt(mean(x^2) + eps) * w, the weight used as stored (not 1 + w). A family whose weights are
stored as an offset from one gives `offset` 1: the kernels then see offset + w."""
from ..kernels import ops
from ..weights import TensorNeed
from .base import Part
from .registry import register


def _around_zero(shape, gen, device, std, norm_std):
    """A random model's weights of a norm that adds its offset itself."""
    import torch
    return norm_std * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


@register("norm", "rmsnorm")
class RMSNorm(Part):
    graph_safe = True
    hands_on = True      # y = x * w / rms(x): a product may apply the 1 / rms to its sums instead (NormedRows)
    takes_scaled_sum = True     # forward(..., delta=, factors=) first adds factors * delta to x (a factor a channel)

    def __init__(self, size, eps, weight, offset=0.0):
        """offset: added to the stored weight (1 for weights stored as offsets from one)."""
        self.size = int(size)
        self.eps = float(eps)
        self.weight_name = weight
        self.offset = float(offset)
        self.w = None

    def tensor_needs(self):
        if self.offset:
            return {self.weight_name: TensorNeed((self.size,), "scale", _around_zero)}
        return {self.weight_name: TensorNeed((self.size,), "scale")}

    def load(self, tensors, rt):
        self.w = rt.weight(tensors[self.weight_name], matrix=False)
        if self.offset:
            self.w = (self.w + self.offset).contiguous()

    def forward(self, ctx, x, rows=None, name="normed", delta=None, factors=None):
        """delta f32 [T, size] with factors f32 [size]: x becomes x + factors * delta first, in place, and that
        sum is normed, in one kernel (no rows then)."""
        n = x.shape[0] if rows is None else rows.shape[0]
        y = ctx.rt.buffer(name, (n, self.size))
        if delta is not None:
            if rows is not None:
                raise ValueError("rmsnorm: rows are not gathered while a sum is added")
            ops.rmsnorm_scaled_sum(x, delta, factors, self.w, y, self.eps)
        else:
            ops.rmsnorm(x, self.w, y, self.eps, rows)
        return y


@register("norm", "layernorm")
class LayerNorm(Part):
    """y = (x - mean) / sqrt(var + eps) * w with var the mean of the squared deviations; a weight and
    no bias. Not of the form x * w / rms(x), so no product can finish it (`hands_on` stays off); what
    it can take on instead is the sum that joins the residual stream just before it
    (`forward(..., delta=, mult=)`: x <- x + mult * delta, then the norm of that, one kernel)."""
    graph_safe = True
    adds_sum = True      # forward(..., delta=, mult=) adds a sum to x on the way

    def __init__(self, size, eps, weight):
        self.size = int(size)
        self.eps = float(eps)
        self.weight_name = weight
        self.w = None

    def tensor_needs(self):
        return {self.weight_name: TensorNeed((self.size,), "scale")}

    def load(self, tensors, rt):
        self.w = rt.weight(tensors[self.weight_name], matrix=False)

    def forward(self, ctx, x, rows=None, name="normed", delta=None, mult=1.0):
        n = x.shape[0] if rows is None else rows.shape[0]
        y = ctx.rt.buffer(name, (n, self.size))
        ops.layernorm(x, self.w, y, self.eps, rows, delta=delta, mult=mult)
        return y

    def forward_in_place(self, ctx, x):
        """x <- norm(x), float32: for a norm that is part of the residual stream itself."""
        ops.layernorm(x, self.w, x, self.eps)
        return x
