"""A token's own input to the residual stream, layer by layer.

A table beside the embedding holds, for every token id, a short row for every layer. At the end of layer i, with
e = that token's row for this layer (columns [i dim, (i + 1) dim) of the table):

    g = gelu_tanh(W_gate x) * e;   y = W_proj g;   x <- x + y / sqrt(mean(y^2) + eps) * w

The gate reads the residual stream x itself, not a normed copy of it. Three small kernels do it (the gate, the
second product, the norm with the sum), in float32 arithmetic; the matrices and the table are kept in the compute
dtype, W_proj transposed so that neighbouring threads read neighbouring weights. In bfloat16 mode a step of many
tokens leaves the gates as bfloat16 and takes the second product to the matrix cores (float32 sums). The table is one
tensor for all layers and is kept on the GPU once.
"""
import torch

from ..kernels import ops
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register


@register("token_input", "gated_table")
class GatedTableInput(Part):
    graph_safe = True

    def __init__(self, hidden_size, vocab_size, dim, layer, layers, eps, names, shared=None):
        """names: table, gate, proj, norm -> tensor names. layer: which of the table's `layers` parts is this one's."""
        self.hidden_size, self.vocab_size, self.dim = int(hidden_size), int(vocab_size), int(dim)
        self.layer, self.layers, self.eps = int(layer), int(layers), float(eps)
        if not 0 <= self.layer < self.layers or self.dim <= 0:
            raise ValueError(f"part {self.layer} of a table of {self.layers} parts of {self.dim}")
        self.names = dict(names)
        self.table = self.gate = self.proj_t = self.norm_w = None

    def tensor_needs(self):
        n = self.names
        return {n["table"]: TensorNeed((self.vocab_size, self.layers * self.dim), "table"),
                n["gate"]: TensorNeed((self.dim, self.hidden_size)),
                n["proj"]: TensorNeed((self.hidden_size, self.dim)),
                n["norm"]: TensorNeed((self.hidden_size,), "scale")}

    def load(self, tensors, rt):
        n = self.names
        self.table = rt.shared_weight(n["table"], tensors[n["table"]])
        proj = rt.weight(tensors[n["proj"]])
        self.gate, self.proj_t = rt.weight(tensors[n["gate"]]), proj.t().contiguous()
        # bfloat16, many tokens, sizes the matrix cores take: the second product is one of theirs
        self.proj = None
        if rt.dtype == torch.bfloat16 and self.dim % 32 == 0 and self.hidden_size % 16 == 0:
            self.proj = Linear(proj, scratch=rt.scratch)
        self.norm_w = rt.weight(tensors[n["norm"]], matrix=False)

    def forward(self, ctx, x):
        T = x.shape[0]
        g = ctx.rt.buffer("token_input_gates", (T, self.dim), torch.float32)
        y = ctx.rt.buffer("token_input_rows", (T, self.hidden_size), torch.float32)
        args = (x, ctx.meta.token_ids, self.table, self.layer * self.dim, self.gate, self.proj_t, self.norm_w, self.eps, g, y)
        if self.proj is not None and T > ops.TOKEN_SIDE_FEW:
            g16 = ctx.rt.buffer("token_input_gates16", (T, self.dim), torch.bfloat16)
            ops.token_side(*args, stage=0, g16=g16)
            self.proj.forward(g16, y)
            ops.token_side(*args, stage=2)
            return
        ops.token_side(*args)
