"""A mixer with a matrix of state a head that decays channel by channel: a gated linear attention.

From the normed rows h:  q = W_q h times dim^-1/2, k = W_k h (heads x dim), v = W_v h (heads x vdim), and a
decay a head and key channel, alpha = sigmoid(z)^(1 / tau) with z = W_a2 (W_a1 h) + b through a narrow middle.
A head keeps S [dim, vdim], zero at the start, and for every token
    S <- diag(alpha) S + k v^T;   o = S^T q         (o sees the token's own write; the decay scales the rows of S)
o is divided by its root mean square over vdim, multiplied by a weight [vdim] that the heads share and by
silu(W_g h), and goes through W_o. The decay from its middle on, the state, the recurrence and the norm a head
are float32 in either mode. What a sequence carries from step to step: S.
"""
import torch

from ..cache import StateNeed
from ..kernels import ops, recurrent
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register


def _second_init(width):
    """The second of two products through a narrow middle, drawn so that the decays of a random model spread
    over (0, 1): pre-activations of about two units (the middle's entries are sums of `width` terms of the
    model's deviation)."""
    def init(shape, gen, device, std, norm_std):
        size = 2.0 / (shape[1] ** 0.5 * max(std, 1e-3) * width ** 0.5)
        return size * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)
    return init


def _bias_init(shape, gen, device, std, norm_std):
    """A decay's bias of a random model: around 2, so that most channels remember for a while."""
    return 2.0 + torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


@register("mixer", "decayed_linear_attention")
class DecayedLinearAttention(Part):
    graph_safe = True
    stores_fresh_rows = True     # its output projection stores into rows that hold nothing yet (StepContext.adds_to)

    def __init__(self, hidden_size, heads, dim, vdim, tau, eps, names, rank=None, shared=None):
        """names: q, k, v, g, a1, a2, a2_bias, norm, o -> tensor names. tau: the decay is sigmoid(.)^(1 / tau).
        eps: of the norm a head. rank: the size of the decay's middle; None: read from the stored tensor."""
        self.hidden_size, self.heads, self.dim, self.vdim = int(hidden_size), int(heads), int(dim), int(vdim)
        self.tau, self.eps = float(tau), float(eps)
        self.rank = None if rank is None else int(rank)
        if self.tau <= 0 or not 0 < self.dim <= recurrent.MAX_KEY_DIM:
            raise ValueError(f"the linear attention takes a positive tau and keys of up to {recurrent.MAX_KEY_DIM}")
        self.names = dict(names)
        self.proj = self.o = None

    def tensor_needs(self):
        n, W = self.names, self.hidden_size
        qk, v = self.heads * self.dim, self.heads * self.vdim
        return {n["q"]: TensorNeed((qk, W)), n["k"]: TensorNeed((qk, W)), n["v"]: TensorNeed((v, W)),
                n["g"]: TensorNeed((v, W)),
                n["a1"]: TensorNeed((self.rank, W)),
                n["a2"]: TensorNeed((qk, self.rank), "matrix", _second_init(W)),
                n["a2_bias"]: TensorNeed((qk,), "bias", _bias_init),
                n["norm"]: TensorNeed((self.vdim,), "scale"),
                n["o"]: TensorNeed((W, v))}

    def cache_need(self):
        return (StateNeed((self.heads, self.dim, self.vdim), torch.float32),)

    def load(self, tensors, rt):
        n = self.names
        # one projection [q | k | v | g | a1]: the rows are read once; q, k and v are read where its float32 sums lie
        rows = [tensors[n[k]].to(rt.device) for k in ("q", "k", "v", "g", "a1")]
        self.proj = Linear(rt.weight(torch.cat(rows, 0)), scratch=rt.scratch)
        qk, v = self.heads * self.dim, self.heads * self.vdim
        self.g_off, self.a_off = 2 * qk + v, 2 * qk + 2 * v
        self.middle = rows[4].shape[0]
        self.width = self.a_off + self.middle
        self.a2 = rt.weight(tensors[n["a2"]])
        self.a2_bias = rt.weight(tensors[n["a2_bias"]], matrix=False)
        self.norm_w = rt.weight(tensors[n["norm"]], matrix=False)
        self.o = Linear(rt.weight(tensors[n["o"]]), scratch=rt.scratch)

    def forward(self, ctx, y, x):
        rt = ctx.rt
        T = y.shape[0]
        state = ctx.cache.state_views(ctx.cache_entry)[0]
        proj = rt.buffer("gla_proj", (T, self.width), torch.float32)
        self.proj.forward(y, proj)
        # the decays: the middle's second product, float32, leaves sigmoid(sum + bias)^(1 / tau) where it stores
        decay = rt.buffer("gla_decay", (T, self.heads * self.dim), torch.float32)
        ops.gemm_plain_columns(proj, self.a_off, self.middle, self.a2, decay,
                               decay=("sigmoid_root", self.a2_bias, 1.0 / self.tau))
        o = rt.buffer("gla_o", (T, self.heads * self.vdim), torch.float32)
        recurrent.gated_delta(proj, None, 0, 0, None, None, state, ctx.meta, o, self.heads, self.heads, self.dim,
                              self.vdim, decay=decay, correction=False, out_scale=self.dim ** -0.5)
        gated = rt.buffer("gla_gated", (T, self.heads * self.vdim))
        recurrent.gated_head_norm(o, proj, self.g_off, self.norm_w, gated, self.heads, self.vdim, self.eps, gate="silu")
        self.o.forward(gated, x, accumulate=ctx.adds_to(x))
