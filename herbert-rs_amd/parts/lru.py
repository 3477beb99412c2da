"""A mixer with one number of state a channel: the real-gated linear recurrent unit between two branches.

From the normed rows h, two branches of `width` channels: g = gelu_tanh(W_y h + b_y) and u = the rows
W_x h + b_x filtered along time, channel by channel, over the token and the K - 1 tokens before it (taps
[width, K], column K - 1 weighs the token itself; nothing precedes a sequence's first token) plus a bias a
channel. u is cut into `blocks` equal parts; in part b, with square matrices [out, in] of the part's size,
    r = sigmoid(R_b u_b + rb_b),   i = sigmoid(I_b u_b + ib_b),
and every channel keeps one number S, zero at the start:
    a = exp(-rate r softplus(lam)),   S <- a S + sqrt(1 - a^2) i u        (the first token is no special case)
The output is W_o (S g). The filter's output, the gates, the decay and the recurrence are float32 in either
mode. What a sequence carries from step to step: S, and the last K - 1 inputs of the filter.
"""
import torch

from ..cache import StateNeed
from ..kernels import ops, recurrent
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register


def _taps_init(shape, gen, device, std, norm_std):
    """Taps near an average of the window, so that a random model's filter passes its input on."""
    return 1.0 / shape[1] + 0.3 * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


def _bias_init(shape, gen, device, std, norm_std):
    return 0.3 * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


def _rate_init(shape, gen, device, std, norm_std):
    """lam of a random model: softplus(lam) between about 0.02 and 0.7, so that memories last from a few to a few
    dozen tokens."""
    return -4.0 + 3.5 * torch.rand(shape, generator=gen, device=device, dtype=torch.float32)


def _gate_init(shape, gen, device, std, norm_std):
    """The gates' square matrices: pre-activations of about unit size for inputs of the model's deviation."""
    return torch.randn(shape, generator=gen, device=device, dtype=torch.float32) / shape[-1] ** 0.5


@register("mixer", "gated_lru")
class GatedLRU(Part):
    graph_safe = True
    stores_fresh_rows = True     # its output projection stores into rows that hold nothing yet (StepContext.adds_to)

    def __init__(self, hidden_size, width, blocks, conv, names, rate=8.0, shared=None):
        """names: x, x_bias, y, y_bias, conv, conv_bias, r, r_bias, i, i_bias, lam, o -> tensor names.
        conv: the filter's taps (1: the token alone). rate: the constant in the decay's exponent."""
        self.hidden_size, self.width, self.blocks, self.taps = int(hidden_size), int(width), int(blocks), int(conv)
        self.rate = float(rate)
        if self.width % self.blocks:
            raise ValueError("the recurrent unit's width must be a multiple of its blocks")
        if not 1 <= self.taps <= recurrent.MAX_TAPS:
            raise ValueError(f"the recurrent unit's filter takes 1 to {recurrent.MAX_TAPS} taps, not {self.taps}")
        self.block = self.width // self.blocks
        self.names = dict(names)
        self.proj = self.o = None

    def tensor_needs(self):
        n, H, W, B, b = self.names, self.hidden_size, self.width, self.blocks, self.block
        return {n["x"]: TensorNeed((W, H)), n["x_bias"]: TensorNeed((W,), "bias", _bias_init),
                n["y"]: TensorNeed((W, H)), n["y_bias"]: TensorNeed((W,), "bias", _bias_init),
                n["conv"]: TensorNeed((W, self.taps), "taps", _taps_init),
                n["conv_bias"]: TensorNeed((W,), "bias", _bias_init),
                n["r"]: TensorNeed((B, b, b), "matrix", _gate_init), n["r_bias"]: TensorNeed((B, b), "bias", _bias_init),
                n["i"]: TensorNeed((B, b, b), "matrix", _gate_init), n["i_bias"]: TensorNeed((B, b), "bias", _bias_init),
                n["lam"]: TensorNeed((W,), "rate", _rate_init),
                n["o"]: TensorNeed((H, W))}

    def cache_need(self):
        needs = [StateNeed((self.width,), torch.float32)]
        if self.taps > 1:
            needs.append(StateNeed((self.taps - 1, self.width), torch.float32))
        return tuple(needs)

    def load(self, tensors, rt):
        n = self.names
        # one projection [x | y]: the rows are read once
        self.proj = Linear(rt.weight(torch.cat([tensors[n["x"]].to(rt.device), tensors[n["y"]].to(rt.device)], 0)),
                           scratch=rt.scratch)
        f32 = lambda k: rt.weight(tensors[n[k]], matrix=False).reshape(-1).contiguous()
        self.x_bias, self.y_bias, self.conv_bias = f32("x_bias"), f32("y_bias"), f32("conv_bias")
        self.r_bias, self.i_bias, self.lam = f32("r_bias"), f32("i_bias"), f32("lam")
        self.conv_w = rt.weight(tensors[n["conv"]], matrix=False)
        # a block's two matrices one above the other: one product a block leaves [r | i] of the block
        r, i = rt.weight(tensors[n["r"]]), rt.weight(tensors[n["i"]])
        self.gate_w = torch.cat([r, i], 1).contiguous()                      # [blocks, 2 block, block]
        self.o = Linear(rt.weight(tensors[n["o"]]), scratch=rt.scratch)

    def forward(self, ctx, y, x):
        rt, W, b = ctx.rt, self.width, self.block
        T = y.shape[0]
        views = ctx.cache.state_views(ctx.cache_entry)
        state = views[0]
        conv_state = views[1] if self.taps > 1 else rt.buffer("lru_no_filter", (1, 1, W), torch.float32)
        proj = rt.buffer("lru_proj", (T, 2 * W), torch.float32)
        self.proj.forward(y, proj)
        ug = rt.buffer("lru_ug", (T, 2 * W), torch.float32)
        recurrent.lru_inputs(proj, self.x_bias, self.y_bias, self.conv_w, self.conv_bias, conv_state, ctx.meta, ug)
        # the gates' pre-activations: a float32 product a block of the block's u with its two matrices
        gates = rt.buffer("lru_gates", (T, 2 * W), torch.float32)
        ops.gemm_plain_batched(ug, self.gate_w, gates, T, 2 * b, b, 2 * W, b, 2 * W, self.blocks, b, 2 * b * b, 2 * b)
        out = rt.buffer("lru_out", (T, W))
        recurrent.lru_scan(ug, gates, self.r_bias, self.i_bias, self.lam, self.rate, state, ctx.meta, out, b)
        self.o.forward(out, x, accumulate=ctx.adds_to(x))
