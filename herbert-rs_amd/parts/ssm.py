"""A mixer with a matrix of state a head and one decay a head: the state-space layer.

From the normed rows h, one projection gives [z | x | B | C | dt] of sizes inner, inner, groups x N, groups x N
and heads (inner = heads x P). x, B and C pass a filter along time, channel by channel, over the token and the
K - 1 tokens before it (taps [channels, K] with a bias; column K - 1 weighs the token itself; nothing precedes a
sequence's first token), then silu. With dt = softplus(dt + dt_bias) a head h (on group h / (heads / groups) of
B and C) keeps S [N, P], zero at the start, and for every token
    S <- exp(-exp(A_log_h) dt) S + dt B x^T;   y = S^T C + D_h x.
The heads' outputs, joined, are multiplied by silu(z), divided by their root mean square in `norm_groups` equal
parts of the row (each part by its own), multiplied by a weight [inner], and go through W_o. Everything from the
projection's sums on is float32 in either mode. What a sequence carries from step to step: S, and the last
K - 1 inputs of the filter.
"""
import torch

from ..cache import StateNeed
from ..kernels import recurrent
from ..weights import TensorNeed
from .base import Part
from .delta import _rate_init, _taps_init
from .linear import Linear
from .registry import register

SECTION, SECTION_FEW = 256, 64        # channels of the filter that one wave takes; where the step has few tokens


def _skip_init(shape, gen, device, std, norm_std):
    """The factors of the input's direct way to the output: around one."""
    return 1.0 + 0.3 * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


def _conv_bias_init(shape, gen, device, std, norm_std):
    return 0.3 * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


@register("mixer", "state_space")
class StateSpace(Part):
    graph_safe = True
    stores_fresh_rows = True     # its output projection stores into rows that hold nothing yet (StepContext.adds_to)

    def __init__(self, hidden_size, heads, vdim, state, groups, conv, eps, names, norm_groups=1, shared=None):
        """names: in, conv, conv_bias, dt_bias, A_log, D, norm, o -> tensor names. conv: the filter's taps (1: none).
        state: rows N of a head's matrix; vdim: its columns P. eps: of the norm in groups."""
        self.hidden_size, self.heads, self.P, self.N = int(hidden_size), int(heads), int(vdim), int(state)
        self.groups, self.taps, self.norm_groups = int(groups), int(conv), int(norm_groups)
        self.eps = float(eps)
        self.names = dict(names)
        if self.heads % self.groups:
            raise ValueError("heads must be divisible by groups")
        if self.inner % self.norm_groups:
            raise ValueError(f"{self.norm_groups} groups of the norm do not divide {self.inner} channels")
        if not 1 <= self.taps <= recurrent.MAX_TAPS or not 0 < self.N <= recurrent.MAX_SSM_STATE:
            raise ValueError(f"the state-space kernels take 1 to {recurrent.MAX_TAPS} taps and a state of up to "
                             f"{recurrent.MAX_SSM_STATE} rows, not {self.taps} and {self.N}")
        self.proj = self.o = None

    @property
    def inner(self):
        return self.heads * self.P

    @property
    def channels(self):
        """Channels that pass the filter: x, B, C."""
        return self.inner + 2 * self.groups * self.N

    @property
    def width(self):
        return 2 * self.inner + 2 * self.groups * self.N + self.heads

    def tensor_needs(self):
        n, W = self.names, self.hidden_size
        return {n["in"]: TensorNeed((self.width, W)),
                n["conv"]: TensorNeed((self.channels, self.taps), "taps", _taps_init),
                n["conv_bias"]: TensorNeed((self.channels,), "bias", _conv_bias_init),
                n["dt_bias"]: TensorNeed((self.heads,), "rate", _rate_init),
                n["A_log"]: TensorNeed((self.heads,), "rate", _rate_init),
                n["D"]: TensorNeed((self.heads,), "rate", _skip_init),
                n["norm"]: TensorNeed((self.inner,), "scale"),
                n["o"]: TensorNeed((W, self.inner))}

    def cache_need(self):
        # (the walk's kernel lays a head's matrix out as its threads hold it)
        needs = [StateNeed((self.heads, recurrent.ssm_state_floats(self.N, self.P)), torch.float32)]
        if self.taps > 1:
            needs.append(StateNeed((self.taps - 1, self.channels), torch.float32))
        return tuple(needs)

    def load(self, tensors, rt):
        n = self.names
        self.proj = Linear(rt.weight(tensors[n["in"]]), scratch=rt.scratch)
        self.conv_w = rt.weight(tensors[n["conv"]], matrix=False)
        self.conv_b = rt.weight(tensors[n["conv_bias"]], matrix=False)
        self.dt_bias = rt.weight(tensors[n["dt_bias"]], matrix=False)
        self.a_log = rt.weight(tensors[n["A_log"]], matrix=False)
        self.d_skip = rt.weight(tensors[n["D"]], matrix=False)
        self.norm_w = rt.weight(tensors[n["norm"]], matrix=False)
        self.o = Linear(rt.weight(tensors[n["o"]]), scratch=rt.scratch)

    def forward(self, ctx, y, x):
        rt = ctx.rt
        T, C = y.shape[0], self.channels
        views = ctx.cache.state_views(ctx.cache_entry)
        proj = rt.buffer("ssm_proj", (T, self.width), torch.float32)
        self.proj.forward(y, proj)
        u = rt.buffer("ssm_xbc", (T, C), torch.float32)
        conv_state = views[1] if self.taps > 1 else rt.buffer("ssm_no_conv", (1, 1, C), torch.float32)
        section = SECTION if T > 64 else SECTION_FEW       # (few tokens: more, shorter waves)
        recurrent.conv_silu(proj, self.conv_w, conv_state, ctx.meta, u, 0, 1, 0, 1.0, 0.0, -(-C // section), section,
                            col0=self.inner, bias=self.conv_b)
        walked = rt.buffer("ssm_y", (T, self.inner), torch.float32)
        recurrent.ssm_scan(u, proj, self.inner + C, self.dt_bias, self.a_log, self.d_skip, views[0], ctx.meta, walked,
                           self.heads, self.groups, self.N, self.P)
        gated = rt.buffer("ssm_gated", (T, self.inner))
        recurrent.gated_group_norm(walked, proj, 0, self.norm_w, gated, self.norm_groups, self.eps)
        adds = ctx.adds_to(x)
        left = ctx.leave_norm(self.o, x) if adds else None
        self.o.forward(gated, x, accumulate=adds, leave=None if left is None else left.leave())
