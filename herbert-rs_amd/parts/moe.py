"""A feed-forward of many small experts, of which each token uses a few.

Router: z = W_r y + b in float32. A token goes to the `top` experts whose z is largest, and weighs them by
exp(z) normalised over those experts alone (not over all of them). An expert: g = min(W_gate y, limit), u = clamp(W_up y, -limit,
limit), out = W_down (g sigmoid(alpha g) (u + 1)), no biases. The part's output is the weighted sum
of the chosen experts' outputs. The routing never reaches the host: the (token, expert) pairs are put
in the order of their experts on the GPU and the experts' products run over a list of row tiles of
fixed length, so a step's grid depends on its size only.

Variants, each a parameter. `routing="scores"`: s = sigmoid(z); the choice runs on s + correction (a stored
vector) and only within the `keep` best of `groups` equal groups of neighbouring experts, a group being worth
the two highest of its selection values, added; the weights are the chosen experts' s over their sum (+ 1e-20).
`activation="silu"`: an expert is W_down (silu(W_gate y) (W_up y)), nothing clamped. `shared_expert`: one more
expert of that form and a width of its own that every token takes, its output times sigmoid(w_sg . y) (one
number a token) added to the routed experts' sum. With routing "scores" three more: `scoring="softmax"` (s is the
softmax of z over all experts instead of its sigmoids), `group_worth=1` (a group is worth its highest selection
value alone), `renormalize=False` (the weights are the chosen experts' s as they are). `identity`: so many
further outputs of the router, behind the experts', stand for experts without matrices, whose output is their
input; they are scored, grouped and chosen with the others.
"""
import math

import torch

from ..kernels import mfma, moe, ops
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register

GATE_ALPHA = 1.702


def _bias_init(shape, gen, device, std, norm_std):
    return 0.1 * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


@register("feed_forward", "routed_experts")
class RoutedExperts(Part):
    graph_safe = True

    def __init__(self, hidden_size, intermediate_size, experts, top, names, limit=None, alpha=GATE_ALPHA, shared=None,
                 routing="softmax", groups=1, keep=1, activation="clamped", shared_expert=None, scoring="sigmoid",
                 group_worth=2, renormalize=True, identity=0):
        """names: router, router_bias (None: none; with routing "scores" it is the correction of the choice),
        and gate, up, down as patterns with {e} for the expert's number.
        shared_expert: None or {"intermediate_size": .., "names": {gate, up, down, sg}}."""
        self.hidden_size, self.inter = int(hidden_size), int(intermediate_size)
        self.experts, self.top = int(experts), int(top)
        if routing not in ("softmax", "scores") or activation not in ("clamped", "silu"):
            raise ValueError(f"routing is 'softmax' or 'scores' and activation 'clamped' or 'silu', not {routing!r} "
                             f"and {activation!r}")
        self.routing, self.groups, self.keep = routing, int(groups), int(keep)
        if scoring not in ("sigmoid", "softmax") or group_worth not in (1, 2):
            raise ValueError(f"scoring is 'sigmoid' or 'softmax' and a group is worth its top 1 or 2, not {scoring!r}, {group_worth!r}")
        self.scoring, self.group_worth, self.renormalize, self.identity = scoring, int(group_worth), bool(renormalize), int(identity)
        if routing != "scores" and (scoring != "sigmoid" or group_worth != 2 or not renormalize or self.identity):
            raise ValueError("softmax scores, a group's worth, weights as they are and experts without matrices go with routing 'scores'")
        if self.identity < 0 or (self.identity and shared_expert is not None):
            raise ValueError("experts without matrices: a count of zero or more, and no shared expert beside them")
        if activation == "silu":
            self.limit, self.alpha, self.shift = math.inf, 1.0, 0.0
        else:
            if limit is None:
                raise ValueError("the clamped activation needs its limit")
            self.limit, self.alpha, self.shift = float(limit), float(alpha), 1.0
        self.names = dict(names)
        if not 0 < self.top <= self.routed or self.routed > moe.MAX_EXPERTS:
            raise ValueError(f"{self.top} of {self.routed} experts (the router takes up to {moe.MAX_EXPERTS})")
        if routing == "scores" and (self.groups <= 0 or self.routed % self.groups or not 0 < self.keep <= self.groups
                                    or self.top > self.keep * (self.routed // self.groups)):
            raise ValueError(f"{self.top} experts cannot come from {self.keep} of {self.groups} groups of "
                             f"{self.routed} experts")
        self.shared_expert = None
        if shared_expert is not None:
            self.shared_expert = (int(shared_expert["intermediate_size"]), dict(shared_expert["names"]))

    @property
    def routed(self):
        """Outputs of the router: the experts and, behind them, the experts without matrices."""
        return self.experts + self.identity

    def tensor_needs(self):
        n, W, F = self.names, self.hidden_size, self.inter
        needs = {n["router"]: TensorNeed((self.routed, W))}
        if n.get("router_bias"):
            needs[n["router_bias"]] = TensorNeed((self.routed,), "bias", _bias_init)
        for e in range(self.experts):
            needs[n["gate"].format(e=e)] = TensorNeed((F, W))
            needs[n["up"].format(e=e)] = TensorNeed((F, W))
            needs[n["down"].format(e=e)] = TensorNeed((W, F))
        if self.shared_expert is not None:
            Fs, sn = self.shared_expert
            needs.update({sn["gate"]: TensorNeed((Fs, W)), sn["up"]: TensorNeed((Fs, W)),
                          sn["down"]: TensorNeed((W, Fs)), sn["sg"]: TensorNeed((1, W))})
        return needs

    def load(self, tensors, rt):
        n = self.names
        router = rt.weight(tensors[n["router"]])
        self.shared_up = self.shared_down = None
        if self.shared_expert is not None:
            # the shared expert's gate is one more row of the router's product (rows up to a multiple of
            # 16, zeros, so that the matrix cores take the product)
            Fs, sn = self.shared_expert
            rows = -(-(self.experts + 1) // 16) * 16
            wide = router.new_zeros((rows, self.hidden_size))
            wide[:self.experts] = router
            wide[self.experts] = rt.weight(tensors[sn["sg"]])[0]
            router = wide
            gate, up = rt.weight(tensors[sn["gate"]]), rt.weight(tensors[sn["up"]])
            self.shared_fused = (rt.dtype == torch.bfloat16 and Fs % 16 == 0 and self.hidden_size % 32 == 0
                                 and mfma.gemm_supported(gate[:1], gate, swiglu=True))
            if self.shared_fused:
                self.shared_up = Linear(mfma.interleave_gate_up(gate, up), scratch=rt.scratch)
            else:
                self.shared_up = Linear(torch.cat([gate, up], 0), scratch=rt.scratch)
            self.shared_down = Linear(rt.weight(tensors[sn["down"]]), scratch=rt.scratch)
        self.router = Linear(router, scratch=rt.scratch)
        self.router_width = router.shape[0]
        self.router_bias = rt.weight(tensors[n["router_bias"]], matrix=False) if n.get("router_bias") else None
        # [E, 2 F, W]: an expert's gate rows, then its up rows; [E, W, F]
        self.gate_up = torch.stack([torch.cat([rt.weight(tensors[n["gate"].format(e=e)]),
                                               rt.weight(tensors[n["up"].format(e=e)])], 0)
                                    for e in range(self.experts)]).contiguous()
        self.down = torch.stack([rt.weight(tensors[n["down"].format(e=e)]) for e in range(self.experts)]).contiguous()
        # bfloat16 with sizes the matrix cores take: the matrices are kept in their operands' order
        W, F = self.hidden_size, self.inter
        self.cores = (rt.dtype == torch.bfloat16 and moe.mfma_takes(W, W, 0, 2 * F) and moe.mfma_takes(F, F, 0, W)
                      and F % 16 == 0)
        if self.cores:
            self.gate_up, self.down = moe.pack_grouped(self.gate_up), moe.pack_grouped(self.down)

    def forward(self, ctx, y, x):
        rt = ctx.rt
        T, E, top, F = y.shape[0], self.routed, self.top, self.inter
        logits = rt.buffer("moe_logits", (T, self.router_width), torch.float32)
        self.router.forward(y, logits)          # float32 sums of the rows' products with the router's matrix
        routing = moe.Routing(rt.buffer("moe_ints", (moe.Routing.ints_needed(T, E, top),), torch.int32),
                              rt.buffer("moe_weight", (T, top), torch.float32), T, E, top, real=self.experts)
        if self.routing == "scores":
            moe.route(logits, self.router_bias, routing, scores=True, groups=self.groups, keep=self.keep,
                      score=self.scoring, worth_top=self.group_worth, renorm=self.renormalize)
        else:
            moe.route(logits, self.router_bias, routing)
        shared = None
        if self.shared_expert is not None:
            Fs = self.shared_expert[0]
            s_act = rt.buffer("moe_shared_act", (T, Fs))
            if self.shared_fused:
                self.shared_up.forward_swiglu(y, s_act)
            else:
                s_gu = rt.buffer("moe_shared_gate_up", (T, 2 * Fs), torch.float32)
                self.shared_up.forward(y, s_gu)
                ops.swiglu(s_gu, s_act)
            shared = rt.buffer("moe_shared_out", (T, self.hidden_size), torch.float32)
            self.shared_down.forward(s_act, shared)
        act = rt.buffer("moe_act", (T * top, F))
        out = rt.buffer("moe_out", (T * top, self.hidden_size), torch.float32)
        if self.cores:
            # matrix cores; the activation is the first product's epilogue
            moe.grouped_mfma(y, self.hidden_size, 0, self.gate_up, act, F, 0, moe.EPI_GLU, routing, gather=True,
                             limit=self.limit, alpha=self.alpha, shift=self.shift)
            moe.grouped_mfma(act, F, 0, self.down, out, self.hidden_size, 0, moe.EPI_F32, routing)
        else:
            gu = rt.buffer("moe_gate_up", (T * top, 2 * F), torch.float32)
            moe.gemm_plain(y, self.gate_up, gu, routing, gather=True)
            moe.activate(gu, act, self.limit, self.alpha, self.shift)
            moe.gemm_plain(act, self.down, out, routing, gather=False)
        moe.combine(out, routing, x, shared=shared, gate=None if shared is None else (logits, E),
                    identity=y if self.identity else None)
