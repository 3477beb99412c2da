"""A token's own input to the residual stream, layer by layer.

A table beside the embedding holds, for every token id, a short row for every layer. At the end of layer i, with
e = that token's row for this layer (columns [i dim, (i + 1) dim) of the table):

    g = gelu_tanh(W_gate x) * e;   y = W_proj g;   x <- x + y / sqrt(mean(y^2) + eps) * w

The gate reads the residual stream x itself, not a normed copy of it. Three small kernels do it (the gate, the
second product, the norm with the sum), in float32 arithmetic in either mode; the matrices and the table are kept in
the compute dtype, W_proj transposed so that neighbouring threads read neighbouring weights. The table is one
tensor for all layers and is kept on the GPU once.
"""
import torch

from ..kernels import ops
from ..weights import TensorNeed
from .base import Part
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
        self.gate, self.proj_t = rt.weight(tensors[n["gate"]]), rt.weight(tensors[n["proj"]]).t().contiguous()
        self.norm_w = rt.weight(tensors[n["norm"]], matrix=False)

    def forward(self, ctx, x):
        T = x.shape[0]
        g = ctx.rt.buffer("token_input_gates", (T, self.dim), torch.float32)
        y = ctx.rt.buffer("token_input_rows", (T, self.hidden_size), torch.float32)
        ops.token_side(x, ctx.meta.token_ids, self.table, self.layer * self.dim, self.gate, self.proj_t, self.norm_w,
                       self.eps, g, y)
