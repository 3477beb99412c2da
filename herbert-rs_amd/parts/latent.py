"""Attention whose keys and values come from one low-rank latent a token.

From the normed rows h: q = W_q h, a head's [dim unrotated | rot_dim rotated]; W_dkv h has kv_rank +
rot_dim rows: the first kv_rank, RMS-normed with a weight, are the latent c, the last rot_dim, rotated,
are one key part that all heads share. Head n's key is [W_uk,n c | that part], its value W_uv,n c; the
score is the dot product of query and key times `scale`, causal, plain softmax; the head's output is
multiplied by sigmoid(W_g h)_n and the heads go through W_o.

What a token leaves in the cache is c and the rotated part, one row of kv_rank + rot_dim numbers, and
no values beside them. The kernels never build a head's keys or values: the query's unrotated part is taken through
W_uk,n^T first (kv_rank numbers), scores and weighted sums then run on the cached rows themselves,
one shared "key head" for all query heads, and the summed latents go through W_uv,n afterwards.
Scores, softmax and the weighted sums are float32 in either mode.

Two parameters change the form. `gate="elementwise"`: W_g has a row for every entry of the joined heads, and
each entry is multiplied by the sigmoid of its own (after W_uv, in a kernel of its own). `pairs=True`: the
rotation turns neighbouring entries (2i, 2i + 1) instead of entries half the rotated size apart; since a score
only ever sees the rotated parts of a query and a key together, the rows of W_q's and W_dkv's rotated parts
are put into the order (even entries, then odd ones) when they are loaded, and the kernels rotate as they do.
"""
import torch

from ..cache import KVNeed
from ..kernels import latent, moe, ops
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register


@register("mixer", "latent_attention")
class LatentAttention(Part):
    graph_safe = True
    stores_fresh_rows = True     # its output projection stores into rows that hold nothing yet (StepContext.adds_to)

    def __init__(self, hidden_size, heads, dim, rot_dim, vdim, kv_rank, scale, eps, position, names, shared=None,
                 gate="head", pairs=False):
        """names: q, dkv, dkv_norm, uk, uv, g (None: no output gate), o -> tensor names. position: the
        spec of a rotation (its rotary_dims <= rot_dim entries of the rotated part are rotated)."""
        self.hidden_size, self.heads = int(hidden_size), int(heads)
        self.dim, self.rot_dim, self.vdim, self.rank = int(dim), int(rot_dim), int(vdim), int(kv_rank)
        self.scale, self.eps = float(scale), float(eps)
        self.names = dict(names)
        self.position = shared.position(position)
        if gate not in ("head", "elementwise"):
            raise ValueError(f"gate is 'head' or 'elementwise', not {gate!r}")
        self.gate_kind, self.pairs = gate, bool(pairs)
        if self.rank > latent.MAX_RANK or self.rot_dim > latent.MAX_ROT:
            raise ValueError(f"the latent attention's kernels take a latent of up to {latent.MAX_RANK} + "
                             f"{latent.MAX_ROT}, not {self.rank} + {self.rot_dim}")

    @property
    def row(self):
        return self.rank + self.rot_dim

    def tensor_needs(self):
        n, W, H = self.names, self.hidden_size, self.heads
        needs = {n["q"]: TensorNeed((H * (self.dim + self.rot_dim), W)), n["dkv"]: TensorNeed((self.row, W)),
                 n["dkv_norm"]: TensorNeed((self.rank,), "scale"), n["uk"]: TensorNeed((H * self.dim, self.rank)),
                 n["uv"]: TensorNeed((H * self.vdim, self.rank)), n["o"]: TensorNeed((W, H * self.vdim))}
        if n.get("g"):
            needs[n["g"]] = TensorNeed((H * self.vdim if self.gate_kind == "elementwise" else H, W))
        return needs

    def cache_need(self):
        return KVNeed(1, self.row, None, values=False)

    def load(self, tensors, rt):
        n, H = self.names, self.heads
        rot = self.position.rotation_rates()
        self.inv_freq, self.rot_dims = (None, 0) if rot is None else rot
        if self.rot_dims > self.rot_dim:
            raise ValueError(f"{self.rot_dims} rotated entries do not fit the rotated part of {self.rot_dim}")
        wq, wdkv = tensors[n["q"]].to(rt.device), tensors[n["dkv"]].to(rt.device)
        if self.pairs and self.rot_dims:
            # the rotated entries in the order (even, odd): the kernels' rotation of entries half the size apart
            # then turns what were neighbours
            order = torch.cat([torch.arange(0, self.rot_dims, 2), torch.arange(1, self.rot_dims, 2),
                               torch.arange(self.rot_dims, self.rot_dim)]).to(rt.device)
            per = self.dim + self.rot_dim
            q_rows = torch.cat([torch.cat([torch.arange(self.dim, device=rt.device), self.dim + order]) + h * per
                                for h in range(H)])
            wq = wq[q_rows]
            wdkv = wdkv[torch.cat([torch.arange(self.rank, device=rt.device), self.rank + order])]
        rows = [wq, wdkv]
        self.gated = bool(n.get("g"))
        if self.gated:
            rows.append(tensors[n["g"]].to(rt.device))
        # one projection [q | latent and shared key part | gate]
        self.proj = Linear(rt.weight(torch.cat(rows, 0)), scratch=rt.scratch)
        self.q_width = H * (self.dim + self.rot_dim)
        self.gate_width = 0 if not self.gated else H * self.vdim if self.gate_kind == "elementwise" else H
        self.width = self.q_width + self.row + self.gate_width
        self.norm_w = rt.weight(tensors[n["dkv_norm"]], matrix=False)
        # W_uk a head, transposed: [H, rank, dim], so that q' = W_uk,n^T q_n is a product with rows of k = dim
        uk = rt.weight(tensors[n["uk"]]).view(H, self.dim, self.rank)
        self.uk_t = uk.transpose(1, 2).contiguous()
        self.uv = rt.weight(tensors[n["uv"]]).view(H, self.vdim, self.rank).contiguous()
        self.o = Linear(rt.weight(tensors[n["o"]]), scratch=rt.scratch)
        # bfloat16 with sizes the matrix cores take: the heads' matrices are kept in their operands' order
        self.cores = (rt.dtype == torch.bfloat16 and moe.mfma_takes(self.dim, H * self.dim, self.dim, self.rank)
                      and moe.mfma_takes(self.rank, H * self.rank, self.rank, self.vdim))
        if self.cores:
            self.uk_t, self.uv = moe.pack_grouped(self.uk_t), moe.pack_grouped(self.uv)

    def forward(self, ctx, y, x):
        rt, H = ctx.rt, self.heads
        T = y.shape[0]
        kv = ctx.cache.kv_view(ctx.cache_entry)
        proj = rt.buffer("latent_proj", (T, self.width), torch.float32)
        self.proj.forward(y, proj)
        q_full = rt.buffer("latent_q_full", (T, H * self.row), torch.float32)
        cores = self.cores
        q_plain = rt.buffer("latent_q_plain", (T, H * self.dim), torch.bfloat16) if cores else None
        latent.latent_write(proj, 0, self.q_width, self.norm_w, q_full, self.inv_freq, ctx.meta, kv, H, self.dim,
                            self.rank, self.rot_dim, self.rot_dims, self.eps, write_cache=ctx.owns_cache,
                            q_plain=q_plain)
        # q'[t, n, :] = W_uk,n^T q[t, n, :dim]: a product a head, all heads in one launch
        if cores:
            moe.grouped_mfma(q_plain, H * self.dim, self.dim, self.uk_t, q_full, H * self.row, self.row, moe.EPI_F32, M=T)
        else:
            ops.gemm_plain_batched(proj, self.uk_t, q_full, T, self.rank, self.dim, self.width, self.dim,
                                   H * self.row, H, self.dim + self.rot_dim, self.rank * self.dim, self.row)
        mixed = rt.buffer("latent_mixed", (T, H * self.rank))
        gate = proj if self.gated and self.gate_kind == "head" else None
        if latent.mfma_takes(kv, self.rank, self.rot_dim):
            latent.latent_attention_mfma(q_full, ctx.meta, kv, mixed, gate, self.q_width + self.row, H, self.rank,
                                         self.rot_dim, self.scale, rt.buffer)
        else:
            latent.latent_attention_plain(q_full, ctx.meta, kv, mixed, gate, self.q_width + self.row, H, self.rank,
                                          self.rot_dim, self.scale)
        # a head's summed latents through its W_uv
        attn = rt.buffer("latent_attn", (T, H * self.vdim))
        if cores:
            moe.grouped_mfma(mixed, H * self.rank, self.rank, self.uv, attn, H * self.vdim, self.vdim, moe.EPI_BF16, M=T)
        else:
            ops.gemm_plain_batched(mixed, self.uv, attn, T, self.vdim, self.rank, H * self.rank, self.rank,
                                   H * self.vdim, H, self.rank, self.vdim * self.rank, self.vdim)
        if self.gated and self.gate_kind == "elementwise":
            gated = rt.buffer("latent_gated", (T, H * self.vdim))
            ops.gate_heads(attn, proj, self.q_width + self.row, gated, H, self.vdim, self.vdim)
            attn = gated
        adds = ctx.adds_to(x)
        left = ctx.leave_norm(self.o, x) if adds else None
        self.o.forward(attn, x, accumulate=adds, leave=None if left is None else left.leave())
