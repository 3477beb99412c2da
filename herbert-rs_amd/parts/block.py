"""How a layer's parts are arranged.

"parallel": with h = norm(x), x += mult * (mixer(h) + feed_forward(h)): one norm, both parts read it,
and their sum joins the residual stream times a constant.

"postnorm": x <- norm_post_mixer(alpha x + mixer(x)); x <- norm_post_ff(alpha x + feed_forward(x)): the parts
take x as it is, and each norm comes after its sum.

"prenorm": x += mixer(norm_input(x)); x += feed_forward(norm_post_mixer(x)), the
arrangement of the reference's two-norm layer
(crates/backends/backend_common/src/generic_layer.rs:1149-1151, 1234-1236,
1246-1248, 1272-1274). With `branch_scale` (not in the reference) each branch is multiplied, channel by
channel, by a learned factor before it joins x, and the layer may have no feed-forward. With `token_input` (not in
the reference either) a part of the category "token_input" adds to x after the layer's other parts, from x itself
and the tokens' ids. A layer may have no feed-forward.
"""
import torch

from ..kernels import ops
from ..weights import TensorNeed
from .base import Part
from .registry import build, register


class ChannelScale(Part):
    """A learned factor a channel on a branch's output, before the branch joins the residual stream."""
    graph_safe = True

    def __init__(self, size, weight):
        self.size = int(size)
        self.weight_name = weight
        self.w = None

    def tensor_needs(self):
        return {self.weight_name: TensorNeed((self.size,), "scale")}

    def load(self, tensors, rt):
        self.w = rt.weight(tensors[self.weight_name], matrix=False)


@register("block", "prenorm")
class PreNormBlock(Part):
    graph_safe = True

    norm_roles = ("input", "post_mixer")

    def __init__(self, mixer, feed_forward, norms, branch_scale=None, token_input=None):
        """branch_scale: None, or {"size": the model's width, "mixer": tensor name, "feed_forward": tensor name}:
        each branch times a stored factor a channel before the sum. Such a block's parts add to float32 rows
        of their own; the kernel of the norm that follows adds them, scaled, to x on its way (the last
        branch of a layer is left for the next layer's first norm, if that is such a block too). Only such
        A block may do without a feed-forward (the reference's layers all have one).
        token_input: None, or the PartSpec of a part of the category "token_input", whose forward(ctx, x) adds to x
        after the mixer and the feed-forward."""
        self.token_input = None if token_input is None else build("token_input", token_input)
        if self.token_input is not None and branch_scale is not None:
            raise ValueError("prenorm block: a token input does not go with scaled branches")
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms
        self.scales = None
        if branch_scale is not None:
            self.scales = {"mixer": ChannelScale(branch_scale["size"], branch_scale["mixer"])}
            if feed_forward is not None:
                self.scales["feed_forward"] = ChannelScale(branch_scale["size"], branch_scale["feed_forward"])
        missing = [r for r in self.norm_roles[:1 if feed_forward is None else 2] if r not in norms]
        if missing:
            raise ValueError(f"prenorm block needs norms {missing}")
        if self.scales is not None:
            for role in self.norm_roles:
                if role in norms and not getattr(norms[role], "takes_scaled_sum", False):
                    raise ValueError("prenorm block: with scaled branches its norms must take a scaled sum on")

    def parts(self):
        parts = [self.norms["input"], self.mixer]
        if self.feed_forward is not None:
            parts += [self.norms["post_mixer"], self.feed_forward]
        if self.scales is not None:
            parts += list(self.scales.values())
        if self.token_input is not None:
            parts.append(self.token_input)
        return parts

    def first_norm(self):
        """The norm that the residual stream meets first in this block."""
        return self.norms["input"]

    def takes_scaled_sum(self):
        """True if this block's first norm adds the scaled branch that the block before left (ctx.pending_scaled)."""
        return self.scales is not None

    def _forward_scaled(self, ctx, x):
        branch = ctx.rt.buffer("branch_sum", tuple(x.shape), torch.float32)
        pending, ctx.pending_scaled = ctx.pending_scaled, None
        if pending is not None and pending[0] == x.data_ptr():
            h = self.norms["input"].forward(ctx, x, delta=pending[1], factors=pending[2])
        else:
            h = self.norms["input"].forward(ctx, x)
        steps = [(self.mixer, self.scales["mixer"])]
        if self.feed_forward is not None:
            steps.append((self.feed_forward, self.scales["feed_forward"]))
        for i, (part, scale) in enumerate(steps):
            ctx.handed = ctx.norm_ahead = ctx.left = None
            # a part that can store its rows instead of adding them says so and finds the rows in ctx.fresh_rows;
            # for any other the rows are cleared first
            if getattr(part, "stores_fresh_rows", False):
                ctx.fresh_rows = branch
            else:
                ops.fill_u32(branch, 0)
            part.forward(ctx, h, branch)
            ctx.fresh_rows = None
            if i + 1 < len(steps):
                h = self.norms["post_mixer"].forward(ctx, x, delta=branch, factors=scale.w)
                continue
            nxt = ctx.next_block
            if isinstance(nxt, PreNormBlock) and nxt.takes_scaled_sum():
                ctx.pending_scaled = (x.data_ptr(), branch, scale.w)
            else:
                ops.rmsnorm_scaled_sum(x, branch, scale.w, None, None, 0.0)

    def forward(self, ctx, x):
        if self.scales is not None:
            self._forward_scaled(ctx, x)
            return
        # (x changes once more after the parts where the block has a token input: nobody prepares the next norm then)
        after = ctx.norm_after_block if self.token_input is None else None
        if self.feed_forward is None:
            self._run(ctx, x, self.norms["input"], self.mixer, after)
        else:
            self._run(ctx, x, self.norms["input"], self.mixer, (self.norms["post_mixer"], ctx.entry))
            self._run(ctx, x, self.norms["post_mixer"], self.feed_forward, after)
        if self.token_input is not None:
            ctx.handed = ctx.norm_ahead = ctx.left = None
            self.token_input.forward(ctx, x)

    @staticmethod
    def _run(ctx, x, norm, part, ahead):
        """part(norm(x)) added to x. A part may offer forward_from_residual(ctx, x, norm), which
        returns True if it has done the norm itself inside its first kernel, or has used what the
        part before left of it (ctx.handed). `ahead` is (the norm that x meets next, its entry)."""
        left, ctx.left = ctx.left, None
        valid = (left is not None and left.norm is norm and left.entry == ctx.entry
                 and left.x.data_ptr() == x.data_ptr() and left.x.shape == x.shape)
        ctx.norm_ahead = ahead
        if valid and left.squares is None:          # the product before has normed the rows as well
            ctx.handed = None
            part.forward(ctx, left.xg, x)
            return
        ctx.handed = left if valid else None
        fused = getattr(part, "forward_from_residual", None)
        if fused is not None and fused(ctx, x, norm):
            return
        ctx.handed = None
        part.forward(ctx, norm.forward(ctx, x), x)


@register("block", "parallel")
class ParallelBlock(Part):
    """x <- x + mult * (mixer(h) + feed_forward(h)) with h = norm(x). The parts add their outputs, as they
    always do, to float32 rows of their own (cleared first) instead of to x. Where the next layer is such
    a block with a norm that can take a sum on, the sum is left for that norm's kernel, which adds it to x
    and norms the result in one pass; otherwise it is added here."""
    graph_safe = True

    norm_roles = ("input",)

    def __init__(self, mixer, feed_forward, norms, mult=1.0, fuse_sum=True):
        self.mixer = mixer
        self.feed_forward = feed_forward
        if "input" not in norms:
            raise ValueError("parallel block needs the norm 'input'")
        self.norm = norms["input"]
        self.mult = float(mult)
        self.fuse_sum = bool(fuse_sum)

    def parts(self):
        return [self.norm, self.mixer] + ([self.feed_forward] if self.feed_forward is not None else [])

    def first_norm(self):
        return self.norm

    def takes_sum(self):
        """True if this block's norm adds a sum that the block before left (ctx.pending_sum)."""
        return self.fuse_sum and getattr(self.norm, "adds_sum", False)

    def forward(self, ctx, x):
        pending, ctx.pending_sum = ctx.pending_sum, None
        if pending is not None and pending[0].data_ptr() == x.data_ptr() and self.takes_sum():
            h = self.norm.forward(ctx, x, delta=pending[1], mult=pending[2])
        else:
            if pending is not None:
                ops.layernorm_free_sum(x, pending[1], pending[2])
            h = self.norm.forward(ctx, x)
        # the two parts' outputs meet in rows of their own (free again: the norm above has taken the sum
        # of the layer before)
        total = ctx.rt.buffer("parallel_sum", tuple(x.shape), torch.float32)
        ctx.handed = ctx.norm_ahead = None
        # a mixer that can store its rows instead of adding them says so (`stores_fresh_rows`) and finds the
        # rows in ctx.fresh_rows; for any other the rows are cleared first
        if getattr(self.mixer, "stores_fresh_rows", False):
            ctx.fresh_rows = total
        else:
            ops.fill_u32(total, 0)
        self.mixer.forward(ctx, h, total)
        ctx.fresh_rows = None
        if self.feed_forward is not None:
            self.feed_forward.forward(ctx, h, total)
        nxt = ctx.next_block
        if isinstance(nxt, ParallelBlock) and nxt.takes_sum():
            ctx.pending_sum = (x, total, self.mult)
        else:
            ops.layernorm_free_sum(x, total, self.mult)


@register("block", "postnorm")
class PostNormBlock(Part):
    """x <- norm_post_mixer(alpha x + mixer(x)), then x <- norm_post_ff(alpha x + feed_forward(x)) (the second
    step only where the layer has a feed-forward). The parts take x as it is, in the compute dtype, and add
    their outputs, as they always do, to float32 rows: rows that already hold alpha x. One kernel between
    two parts norms those rows into x, writes the copy that the next part reads and alpha x where it adds;
    the one after a layer's last part does so for the next layer too, if that is such a block."""
    graph_safe = True

    norm_roles = ("post_mixer", "post_ff")

    def __init__(self, mixer, feed_forward, norms, alpha=1.0):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms
        self.alpha = float(alpha)
        missing = [r for r in self.norm_roles[:1 if feed_forward is None else 2] if r not in norms]
        if missing:
            raise ValueError(f"postnorm block needs norms {missing}")
        if self.alpha == 0.0:
            raise ValueError("postnorm block: alpha must not be zero")
        for role in self.norm_roles:
            if role in norms and not getattr(norms[role], "hands_on", False):
                raise ValueError("postnorm block: its norms are of the form x * w / rms(x)")

    def parts(self):
        parts = [self.mixer, self.norms["post_mixer"]]
        if self.feed_forward is not None:
            parts += [self.feed_forward, self.norms["post_ff"]]
        return parts

    def forward(self, ctx, x):
        rt = ctx.rt
        shape = tuple(x.shape)
        acc = rt.buffer("postnorm_sum", shape, torch.float32)
        y = None if rt.exact else rt.buffer("postnorm_rows", shape)       # (float32: the parts take x as it is)
        pending, ctx.pending_post = ctx.pending_post, None
        if pending != (x.data_ptr(), self.alpha):
            ops.postnorm(x, None, None, y, 0.0, self.alpha, acc=acc)
        nxt = ctx.next_block
        alpha_after = nxt.alpha if isinstance(nxt, PostNormBlock) else 0.0
        steps = [(self.mixer, self.norms["post_mixer"])]
        if self.feed_forward is not None:
            steps.append((self.feed_forward, self.norms["post_ff"]))
        for i, (part, norm) in enumerate(steps):
            ctx.handed = ctx.norm_ahead = ctx.left = ctx.fresh_rows = None
            part.forward(ctx, x if y is None else y, acc)
            last = i + 1 == len(steps)
            ops.postnorm(acc, norm.w, x, None if last and alpha_after == 0.0 else y, norm.eps,
                         alpha_after if last else self.alpha)
        if alpha_after != 0.0:
            ctx.pending_post = (x.data_ptr(), alpha_after)
