"""Grouped-query attention over the paged cache.

Formulas as the reference computes them (`bc/` = crates/backends/backend_common/src/):
q, k, v projections without bias (bc/generic_attention/prefill/mod.rs:73-77),
optional RMSNorm of every head with one weight [head_dim]
(bc/generic_attention/mod.rs:62-76), rotation at absolute positions
(prefill/mod.rs:189-210), keys and values appended to the cache (:232), scores
scaled by 1/sqrt(head_dim) (bc/generic_attention/decode.rs:126), consecutive
query heads sharing a kv head (decode.rs:131-140), causal by count
(prefill/kernel_f32.rs:65-67), output projection added to the residual
(prefill/mod.rs:293, bc/generic_layer.rs:1234-1236).
A window (keys of the last `window` positions only) is a parameter that the
reference does not have. Nor are these: values of another size than the keys
(`value_dim`), a per-head norm without weights (`qk_norm="plain"`), and a query
that grows with the logarithm of its position (`q_temp=(coef, every)`: times
1 + coef ln(floor((p + 1) / every) + 1) at position p, after norm and rotation).

A further form of the part (not in the reference either), taken where any of these is asked for: `conv` (queries,
keys and values pass a filter along time, channel by channel, directly after their projections; the last
conv - 1 projected rows of a sequence are state beside its keys and values), `qk_norm="whole"` (queries, and keys,
are normed over the whole projection at once, before they are split into heads, with a weight of that size),
a position of the kind "rope_pairs" (neighbouring pairs turn), `sink` (the softmax's denominator of a head also
holds exp(s_h), a stored number a head without key or value), `gate` (the joined heads times sigmoid(W_g y)
before the output projection), `bias` (q, k, v and the output projection have biases), `chunk` (a query sees
the keys of its own chunk of that many positions only, the chunks counted from the sequence's start),
`softcap` (a scaled score s becomes softcap tanh(s / softcap) before the softmax). Such a part filters, norms
(over the whole projection, or head by head with weights that all heads share), rotates and writes the cache in
one kernel of its own; rotation and values of another size than the keys go together there.

The kernels keep one head size for queries, keys and values. Where a model's
key and value sizes differ, or where the matrix cores (heads of 32, 64, 128)
would otherwise refuse a head, the part runs them at a larger size whose
further entries are zeros: zero rows of the projections, zero columns of the
output projection. Zeros change no score and no weighted sum; the norm's mean
over the true size d instead of the kept size s is the same as a mean over s
with eps d / s, times sqrt(d / s) a vector, so the score scale takes d / s.
"""
import math

import torch

from ..cache import KVNeed, StateNeed
from ..kernels import mfma, ops, recurrent
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register


def _taps_init(shape, gen, device, std, norm_std):
    """Taps near an average of the window, so that a random model's filter passes its input on."""
    return 1.0 / shape[1] + 0.3 * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


def _bias_init(shape, gen, device, std, norm_std):
    """Biases of a random model: large enough beside the projections' sums that leaving one out shows."""
    return 0.5 * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


def _sink_init(shape, gen, device, std, norm_std):
    """Sinks of a random model: around zero, so that they take a visible share of a short row's weight."""
    return torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


@register("mixer", "attention")
class Attention(Part):
    graph_safe = True

    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, eps, position, names,
                 qk_norm=True, window=None, scale=None, shared=None, reads_cache_only=False,
                 value_dim=None, q_temp=None, conv=None, sink=False, gate=False, bias=False, chunk=None,
                 softcap=None):
        """names: dict with q, k, v, o (and q_norm, k_norm when qk_norm is True or "whole"; q_conv, k_conv, v_conv
        with conv; sink with sink; g with gate; q_bias, k_bias, v_bias, o_bias with bias) -> tensor names.
        qk_norm: True (a weight [head_dim] each for queries and keys), "plain" (no weights), "whole" (over all
        heads of a token at once, weights of that size) or False.
        conv: taps of a filter along time on queries, keys and values (None: none).
        reads_cache_only: the part has no k / v projections and attends over a cache that
        another entry of the schedule fills."""
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be divisible by num_kv_heads")
        if qk_norm not in (True, False, "plain", "whole"):
            raise ValueError(f"qk_norm is True, False, 'plain' or 'whole', not {qk_norm!r}")
        self.hidden_size = int(hidden_size)
        self.nq = int(num_heads)
        self.nkv = int(num_kv_heads)
        self.dim = int(head_dim)                                       # of a query and a key, as stored
        self.vdim = int(value_dim) if value_dim else self.dim          # of a value, as stored
        self.hd = max(self.dim, self.vdim)                             # as kept (load may choose a larger one)
        self.eps = float(eps)
        self.qk_norm = qk_norm
        self.window = int(window) if window else None
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.dim)
        self.q_temp = None if q_temp is None else (float(q_temp[0]), int(q_temp[1]))
        if self.q_temp is not None and self.q_temp[1] <= 0:
            raise ValueError("q_temp = (coef, every) with every a positive number of positions")
        self.names = dict(names)
        self.reads_cache_only = bool(reads_cache_only)
        self.position = shared.position(position)
        self.qkv = self.o = self.q_norm_w = self.k_norm_w = None
        self.taps = int(conv) if conv else 0
        self.sink, self.gate, self.bias = bool(sink), bool(gate), bool(bias)
        self.chunk = int(chunk) if chunk else None
        self.softcap = float(softcap) if softcap else None
        if self.chunk is not None and (self.chunk <= 0 or self.window):
            raise ValueError("chunk is a positive number of positions and does not go with a window")
        if self.softcap is not None and self.softcap <= 0:
            raise ValueError("softcap must be positive")
        self.sink_w = self.taps_w = self.bias_w = self.o_bias_w = None
        # the form with a kernel of its own before the attention (see the module's text)
        self.prepared = bool(self.taps or self.sink or self.gate or qk_norm == "whole" or self.bias or self.chunk
                             or self.softcap or hasattr(self.position, "pair_rates"))
        if self.prepared:
            if self.reads_cache_only or self.q_temp is not None or qk_norm == "plain" or \
                    self.position.rotation() is not None:
                raise ValueError("a filter, a norm over the whole projection, a rotation of pairs, a sink, a gate, "
                                 "biases, chunks or capped scores go with a cache of the part's own, no norm without "
                                 "weights, no growing query and no rotation of halves")
            if self.taps > recurrent.MAX_TAPS:
                raise ValueError(f"the filter takes up to {recurrent.MAX_TAPS} taps, not {self.taps}")
            self.stores_fresh_rows = True        # its output projection stores into rows that hold nothing yet

    @property
    def q_dim(self):
        return self.nq * self.hd

    @property
    def kv_dim(self):
        return self.nkv * self.hd

    # what the kernels are told where the kept size is larger than the keys' own (see the module's text)
    @property
    def kernel_eps(self):
        return self.eps * self.dim / self.hd

    @property
    def kernel_scale(self):
        return self.scale * self.dim / self.hd if self.qk_norm else self.scale

    @property
    def channels(self):
        """Channels that pass the filter: queries, keys, values."""
        return (self.nq + self.nkv) * self.dim + self.nkv * self.vdim

    def tensor_needs(self):
        n, W = self.names, self.hidden_size
        needs = {n["q"]: TensorNeed((self.nq * self.dim, W)),
                 n["o"]: TensorNeed((W, self.nq * self.vdim))}
        if self.qk_norm == "whole":
            needs[n["q_norm"]] = TensorNeed((self.nq * self.dim,), "scale")
            needs[n["k_norm"]] = TensorNeed((self.nkv * self.dim,), "scale")
        if self.taps:
            for key, rows in (("q_conv", self.nq * self.dim), ("k_conv", self.nkv * self.dim), ("v_conv", self.nkv * self.vdim)):
                needs[n[key]] = TensorNeed((rows, self.taps), "taps", _taps_init)
        if self.sink:
            needs[n["sink"]] = TensorNeed((self.nq,), "bias", _sink_init)
        if self.gate:
            needs[n["g"]] = TensorNeed((self.nq * self.vdim, W))
        if self.bias:
            needs[n["q_bias"]] = TensorNeed((self.nq * self.dim,), "bias", _bias_init)
            needs[n["k_bias"]] = TensorNeed((self.nkv * self.dim,), "bias", _bias_init)
            needs[n["v_bias"]] = TensorNeed((self.nkv * self.vdim,), "bias", _bias_init)
            needs[n["o_bias"]] = TensorNeed((W,), "bias", _bias_init)
        if not self.reads_cache_only:
            needs[n["k"]] = TensorNeed((self.nkv * self.dim, W))
            needs[n["v"]] = TensorNeed((self.nkv * self.vdim, W))
        if self.qk_norm is True:
            needs[n["q_norm"]] = TensorNeed((self.dim,), "scale")
            if not self.reads_cache_only:
                needs[n["k_norm"]] = TensorNeed((self.dim,), "scale")
        return needs

    def _kept_size(self, rt):
        """The head size the kernels run at: the larger of keys and values, and in bfloat16 the next size
        that the matrix cores take, unless the rotation or a cache that another entry fills forbids it."""
        size = max(self.dim, self.vdim)
        if self.prepared:
            if rt.dtype == torch.bfloat16:
                for takes in mfma.ATTENTION_HEAD_DIMS:
                    if size <= takes:
                        return takes
            return size
        if self.position.rotation() is not None or self.reads_cache_only:
            if self.vdim != self.dim:
                raise ValueError("values of another size than the keys go with no rotation and a cache of the part's own")
            return size
        if rt.dtype == torch.bfloat16:
            for takes in mfma.ATTENTION_HEAD_DIMS:
                if size <= takes:
                    return takes
        return size

    @staticmethod
    def _heads_padded(w, heads, size, kept, rows=True):
        """[heads x size, W] -> [heads x kept, W] with zero rows behind every head (rows False: the same
        for the columns of [W, heads x size])."""
        if size == kept:
            return w
        if rows:
            out = w.new_zeros((heads, kept, w.shape[1]))
            out[:, :size] = w.view(heads, size, w.shape[1])
            return out.view(heads * kept, w.shape[1])
        out = w.new_zeros((w.shape[0], heads, kept))
        out[:, :, :size] = w.view(w.shape[0], heads, size)
        return out.view(w.shape[0], heads * kept)

    def cache_need(self):
        if self.reads_cache_only:
            return None
        if self.taps > 1:
            return (KVNeed(self.nkv, self.hd, self.window), StateNeed((self.taps - 1, self.channels), torch.float32))
        return KVNeed(self.nkv, self.hd, self.window)

    def _load_prepared(self, tensors, rt):
        n = self.names
        self.hd = self._kept_size(rt)
        # one fused projection [q | k | v | gate], the heads at their own sizes: the kernel that follows reads
        # its float32 sums where they lie and keeps the heads at the size the attention runs at
        rows = [tensors[n[k]].to(rt.device) for k in ("q", "k", "v") + (("g",) if self.gate else ())]
        self.qkv = Linear(rt.weight(torch.cat(rows, 0)), scratch=rt.scratch)
        self.proj_width = self.channels + (self.nq * self.vdim if self.gate else 0)
        self.o = Linear(rt.weight(tensors[n["o"]]), scratch=rt.scratch)
        if self.qk_norm in ("whole", True):
            self.q_norm_w = rt.weight(tensors[n["q_norm"]], matrix=False)
            self.k_norm_w = rt.weight(tensors[n["k_norm"]], matrix=False)
        if self.bias:
            self.bias_w = torch.cat([rt.weight(tensors[n[k]], matrix=False) for k in ("q_bias", "k_bias", "v_bias")],
                                    0).contiguous()
            self.o_bias_w = rt.weight(tensors[n["o_bias"]], matrix=False)
        if self.taps:
            self.taps_w = torch.cat([rt.weight(tensors[n[k]], matrix=False) for k in ("q_conv", "k_conv", "v_conv")],
                                    0).contiguous()
        if self.sink:
            self.sink_w = rt.weight(tensors[n["sink"]], matrix=False)

    def _forward_prepared(self, ctx, y, x):
        rt = ctx.rt
        T = x.shape[0]
        kv = ctx.cache.kv_view(ctx.cache_entry)
        proj = rt.buffer("attn_proj", (T, self.proj_width), torch.float32)
        self.qkv.forward(y, proj)
        q = rt.buffer("q", (T, self.q_dim))
        state = ctx.cache.state_views(ctx.cache_entry)[0] if self.taps > 1 else None
        rates, rot_dims = self.position.pair_rates() if hasattr(self.position, "pair_rates") else (None, 0)
        ops.filter_norm_rotate_write(proj, self.taps_w, state, self.q_norm_w, self.k_norm_w, rates, rot_dims, ctx.meta,
                                     kv, q, self.nq, self.nkv, self.dim, self.vdim, self.hd, self.eps, bias=self.bias_w,
                                     head_norm=self.qk_norm is True)
        attn = rt.buffer("attn", (T, self.q_dim))
        self.attend(ctx, q, kv, attn)
        # the heads leave at their own size, each entry times its gate
        gated = attn
        if self.gate or self.hd != self.vdim:
            gated = rt.buffer("attn_gated", (T, self.nq * self.vdim))
            ops.gate_heads(attn, proj if self.gate else None, self.channels, gated, self.nq, self.hd, self.vdim)
        self.o.forward(gated, x, accumulate=ctx.adds_to(x))
        if self.o_bias_w is not None:
            ops.add_bias(x, self.o_bias_w)

    def load(self, tensors, rt):
        if self.prepared:
            self._load_prepared(tensors, rt)
            return
        n = self.names
        self.hd = kept = self._kept_size(rt)
        rows = [self._heads_padded(tensors[n["q"]].to(rt.device), self.nq, self.dim, kept)]
        if not self.reads_cache_only:
            rows += [self._heads_padded(tensors[n["k"]].to(rt.device), self.nkv, self.dim, kept),
                     self._heads_padded(tensors[n["v"]].to(rt.device), self.nkv, self.vdim, kept)]
        # one fused projection [q rows | k rows | v rows]: the activations are read once
        self.qkv = Linear(rt.weight(torch.cat(rows, 0)), scratch=rt.scratch)
        self.o = Linear(rt.weight(self._heads_padded(tensors[n["o"]].to(rt.device), self.nq, self.vdim, kept, rows=False)),
                        scratch=rt.scratch)
        if self.qk_norm is True:
            pad = lambda w: torch.nn.functional.pad(w, (0, kept - self.dim), value=1.0).contiguous()
            self.q_norm_w = pad(rt.weight(tensors[n["q_norm"]], matrix=False))
            if not self.reads_cache_only:
                self.k_norm_w = pad(rt.weight(tensors[n["k_norm"]], matrix=False))
        elif self.qk_norm == "plain":
            self.q_norm_w = self.k_norm_w = torch.ones(kept, dtype=torch.float32, device=rt.device)

    def forward_from_residual(self, ctx, x, norm):
        """With few rows and bfloat16 weights no norm kernel runs: the projection takes what the
        product before left of the norm, or else does the norm itself on the way."""
        if self.prepared:
            return False
        handed = ctx.take_handed(self.qkv, x)
        if handed is not None:
            self.forward(ctx, handed.xg, x, row_scale=handed.row_scale())
            return True
        if not (hasattr(norm, "w") and hasattr(norm, "eps") and self.qkv.fuses_norm(x)):
            return False
        self.forward(ctx, None, x, fused_norm=norm)
        return True

    def project_out(self, ctx, attn, x):
        """x += attn @ Wo^T, the part's last product into the residual stream."""
        left = ctx.leave_norm(self.o, x)
        self.o.forward(attn, x, accumulate=True, leave=None if left is None else left.leave())

    def forward(self, ctx, y, x, fused_norm=None, row_scale=None):
        if self.prepared:
            self._forward_prepared(ctx, y, x)
            return
        rt = ctx.rt
        T = x.shape[0]
        kv = ctx.cache.kv_view(ctx.cache_entry)
        write_kv = not self.reads_cache_only
        width = self.q_dim + (2 * self.kv_dim if write_kv else 0)
        rot = self.position.rotation()
        cos, sin, rot_dims = rot if rot is not None else (None, None, 0)
        if write_kv and fused_norm is None and row_scale is None and rt.dtype == torch.bfloat16:
            if self.q_temp is None and mfma.gemm_qkv_fusable(y, self.qkv.weight, ctx.meta, kv, self.nq, self.nkv,
                                                             self.hd, rot_dims):
                # a long prompt: the projection norms, rotates and writes the cache in its epilogue
                q = rt.buffer("q", (T, self.q_dim))
                mfma.gemm_qkv(y, self.qkv.weight, self.qkv.packed, self.q_norm_w, self.k_norm_w, cos, sin, ctx.meta,
                              kv, q, self.nq, self.nkv, self.hd, self.kernel_eps)
                attn = rt.buffer("attn", (T, self.q_dim))
                self.attend(ctx, q, kv, attn)
                self.project_out(ctx, attn, x)
                return
        qkv = rt.buffer("qkv", (T, width), torch.float32)
        fused_decode = False
        if write_kv and rt.dtype == torch.bfloat16:
            fused_decode = mfma.decode_fusable(ctx.meta, kv, self.nq, self.nkv, self.hd, rot_dims, rt.dtype)
        slices = None
        if fused_norm is not None:
            self.qkv.forward_normed(x, fused_norm.w, fused_norm.eps, qkv)
        else:
            # (the fused decode kernel of heads of 128 and the rotation kernel of bfloat16 prompts add
            # up slices of K themselves)
            defer = (fused_decode and self.hd == 128) or (not fused_decode and ops.rope_write_adds_slices(
                T, self.hd, rot_dims, rt.dtype, write_kv, cos is not None))
            slices = self.qkv.forward(y, qkv, row_scale=row_scale, defer_slices=defer)
        attn = rt.buffer("attn", (T, self.q_dim))
        if fused_decode:
            # one token a sequence: norm, rotation, cache write and attention in one kernel
            mfma.attention_decode_fused(qkv, self.q_norm_w, self.k_norm_w, cos, sin, ctx.meta, kv, attn,
                                        self.nq, self.nkv, self.hd, self.kernel_eps, self.kernel_scale, self.window,
                                        qkv_slices=slices, scratch=rt.scratch, q_temp=self.q_temp)
            self.project_out(ctx, attn, x)
            return
        q = rt.buffer("q", (T, self.q_dim))
        ops.qk_norm_rope_write(qkv, self.q_norm_w, self.k_norm_w, cos, sin, rot_dims, ctx.meta, kv, q,
                               self.nq, self.nkv, self.hd, self.kernel_eps, write_kv=write_kv, qkv_slices=slices,
                               q_temp=self.q_temp)
        self.attend(ctx, q, kv, attn)
        self.project_out(ctx, attn, x)

    def attend(self, ctx, q, kv, out):
        scale = self.scale if self.prepared else self.kernel_scale
        if q.dtype == torch.bfloat16:
            if mfma.attention_supported(q, kv, self.nq, self.nkv, self.hd):
                mfma.attention(q, ctx.meta, kv, out, self.nq, self.nkv, self.hd, scale, self.window,
                               scratch=ctx.rt.scratch, sinks=self.sink_w, chunk=self.chunk, softcap=self.softcap)
                return
        ops.attention_plain(q, ctx.meta, kv, out, self.nq, self.nkv, self.hd, scale, self.window, sinks=self.sink_w,
                            chunk=self.chunk, softcap=self.softcap)
