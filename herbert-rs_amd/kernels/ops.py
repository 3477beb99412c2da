"""Host side of every kernel: operand checks, then the launch.

Each function checks on the host that shapes, dtypes, devices and layouts are
what the kernel and its grid assume, and only then launches on the current
HIP stream. There is no fallback of any kind behind them.

The operations are those of the reference's op trait (crates/backends/backend_common/src/linear_ops.rs:68-437:
matmul, rms_norm, swiglu, rotation) and of its GPU command buffer
(crates/backends/backend_vulkan/src/backend.rs:182-281: embedding, norms, per-head norms, rotation, cache
append, attention, residual sums), several of them to a kernel here.
"""
import threading

import torch

from ..errors import BackendError
from . import lib

F32 = 0
BF16 = 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(t):
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise BackendError(f"dtype {t.dtype} is not supported by the kernels") from None


_scoped = threading.local()      # .stream: the stream of the forward pass that this thread is in


class stream_scope:
    """While a forward pass runs, the launches go to the stream that was current when it began:
    looking the stream up costs as much as a launch does. A thread has its own."""

    def __enter__(self):
        self.outer = getattr(_scoped, "stream", None)
        _scoped.stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        _scoped.stream = self.outer
        return False


def _stream():
    s = getattr(_scoped, "stream", None)
    return s if s is not None else torch.cuda.current_stream().cuda_stream


def _check(t, name, dtype=None, shape=None):
    """Refuse what a kernel must not be given: not a contiguous GPU tensor, another dtype, another
    shape (None in `shape`: any size). Called for every operand of every launch, hence the short
    way through for what is right."""
    try:
        if t.is_cuda and t.is_contiguous() and (dtype is None or t.dtype == dtype):
            if shape is None or t.shape == shape:
                return
            got = t.shape
            if len(shape) == len(got) and all(s is None or s == d for s, d in zip(shape, got)):
                return
    except AttributeError:
        pass
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise BackendError(f"{name} must be a tensor on the GPU")
    if not t.is_contiguous():
        raise BackendError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise BackendError(f"{name} must be {dtype}, got {t.dtype}")
    raise BackendError(f"{name} must have shape {list(shape)}, got {list(t.shape)}")


def _ptr(t):
    return None if t is None else t.data_ptr()


def embed(ids, table, out, packed=False):
    """out[t, :] = table[ids[t], :] as float32. ids int32 [T], table [V, H], out f32 [T, H].
    packed: the table is stored in the MFMA kernels' order ([H / 32, V / 16, 64, 8])."""
    T = ids.shape[0]
    _check(ids, "ids", torch.int32, (T,))
    _check(table, "table", None, (None, None))
    H = table.shape[1]
    _check(out, "out", torch.float32, (T, H))
    lib.call("elementwise", "hb_embed", ids.data_ptr(), table.data_ptr(), dtype_code(table),
             out.data_ptr(), T, H, table.shape[0], 1 if packed else 0, _stream())


def rmsnorm(x, weight, out, eps, rows=None):
    """out[r] = rmsnorm(x[rows[r]] or x[r]) * weight. x f32 [T, H], weight f32 [H]."""
    _check(x, "x", torch.float32, (None, None))
    H = x.shape[1]
    _check(weight, "weight", torch.float32, (H,))
    if rows is not None:
        _check(rows, "rows", torch.int32, (None,))
        R = rows.shape[0]
    else:
        R = x.shape[0]
    _check(out, "out", None, (R, H))
    lib.call("elementwise", "hb_rmsnorm", x.data_ptr(), weight.data_ptr(), out.data_ptr(),
             dtype_code(out), _ptr(rows), R, H, float(eps), _stream())


def gemm_plain(a, w, c, accumulate=False):
    """c[M, N] (+)= a[M, K] @ w[N, K]^T in float32 arithmetic, any of f32 / bf16 storage."""
    _check(a, "a", None, (None, None))
    _check(w, "w", None, (None, None))
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise BackendError(f"gemm: a is [{M}, {K}] but w is {list(w.shape)}")
    _check(c, "c", None, (M, N))
    if accumulate and c.dtype != torch.float32:
        raise BackendError("gemm: accumulation needs a float32 output")
    lib.call("gemm_plain", "hb_gemm_plain", a.data_ptr(), dtype_code(a), w.data_ptr(), dtype_code(w),
             c.data_ptr(), dtype_code(c), M, N, K, K, K, N, 1 if accumulate else 0, _stream())


def _check_paged(meta, cache, T):
    _check(meta.positions, "positions", torch.int32, (T,))
    _check(meta.seq_of, "seq_of", torch.int32, (T,))
    _check(meta.slots, "slots", torch.int32, (None,))
    _check(cache.page_table, "page_table", torch.int32, (None, None))
    _check(cache.k, "key pages", None, (None, None, cache.page_size, None))
    pages, nkv, page, hd = cache.k.shape
    _check(cache.v, "value pages", cache.k.dtype, (pages, nkv, hd, page))


ROPE_WRITE_SLICES = (2, 4, 8)


def rope_write_adds_slices(T, hd, rot_dims, dtype, write_kv, has_rotation):
    """True if qk_norm_rope_write can add up K slices of the projection itself for such a step: the
    kernel for bfloat16 prompts of 64 tokens or more does."""
    return (dtype == torch.bfloat16 and write_kv and T >= 64 and hd <= 128 and hd % 8 == 0
            and (not has_rotation or rot_dims == hd))


def query_temperature_args(q_temp):
    """(coef, every) as the kernels take them; None: (0, 0), no factor."""
    if q_temp is None:
        return 0.0, 0
    coef, every = float(q_temp[0]), int(q_temp[1])
    if every <= 0:
        raise BackendError("a query's factor grows every so many positions: that number must be positive")
    return coef, every


def qk_norm_rope_write(qkv, q_norm_w, k_norm_w, cos, sin, rot_dims, meta, cache, q_out, nq, nkv, hd, eps,
                       write_kv=True, qkv_slices=None, q_temp=None):
    """Per-head norm (if weights given), rotation (if tables given), q to q_out, k / v to the pages.

    qkv f32 [T, (nq + 2 nkv) hd] (query heads only when write_kv is false); cos / sin f32 [max_pos, rot_dims / 2]; q_out [T, nq hd] in the
    cache's dtype; cache.k / cache.v [pages, nkv, page_size, hd].
    qkv_slices = (slices, pointer, floats between two), as kernels.mfma.gemm(..., defer_slices=True)
    returns it: the projection's sums still lie in that many slices (see rope_write_adds_slices),
    and qkv itself is not read. q_temp = (coef, every): a query at position p is multiplied by
    1 + coef ln(floor((p + 1) / every) + 1) after its norm and rotation.
    """
    coef, every = query_temperature_args(q_temp)
    T = qkv.shape[0]
    _check(qkv, "qkv", torch.float32, (T, (nq + (2 * nkv if write_kv else 0)) * hd))
    _check_paged(meta, cache, T)
    _check(q_out, "q_out", cache.k.dtype, (T, nq * hd))
    if tuple(cache.k.shape[1:]) != (nkv, cache.page_size, hd):
        raise BackendError(f"cache pages {list(cache.k.shape)} do not fit {nkv} kv heads of {hd}")
    for w, name in ((q_norm_w, "q_norm"), (k_norm_w, "k_norm")):
        if w is not None:
            _check(w, name, torch.float32, (hd,))
    if cos is not None:
        _check(cos, "cos", torch.float32, (None, rot_dims // 2))
        _check(sin, "sin", torch.float32, tuple(cos.shape))
        if meta.max_position >= cos.shape[0]:
            raise BackendError(f"position {meta.max_position} beyond the rotation table "
                               f"({cos.shape[0]} rows)")
    n_slices, src, stride = qkv_slices if qkv_slices is not None else (1, qkv.data_ptr(), 0)
    if n_slices > 1 and (n_slices not in ROPE_WRITE_SLICES or stride < qkv.numel() or not rope_write_adds_slices(
            T, hd, rot_dims, q_out.dtype, write_kv, cos is not None)):
        raise BackendError(f"qk_norm_rope_write does not add up {n_slices} slices of the projection here")
    lib.call("elementwise", "hb_qk_norm_rope_write", src, qkv.shape[1], _ptr(q_norm_w),
             _ptr(k_norm_w), _ptr(cos), _ptr(sin), rot_dims, meta.positions.data_ptr(),
             meta.seq_of.data_ptr(), meta.slots.data_ptr(), cache.page_table.data_ptr(),
             cache.page_table.shape[1], cache.page_size, q_out.data_ptr(), cache.k.data_ptr(),
             cache.v.data_ptr(), dtype_code(q_out), T, nq, nkv, hd, float(eps), 1 if write_kv else 0,
             n_slices, stride, coef, every, _stream())


def attention_plain(q, meta, cache, out, nq, nkv, hd, scale, window, sinks=None, chunk=None, softcap=None):
    """Causal (and windowed) attention of every token over its slot's pages. sinks f32 [nq]: the softmax's
    denominator of head h also holds exp(sinks[h]). chunk: a query sees the keys of its own chunk of that many
    positions only (counted from the sequence's start; not together with a window). softcap: a scaled score s
    becomes softcap tanh(s / softcap)."""
    T = q.shape[0]
    if sinks is not None:
        _check(sinks, "sinks", torch.float32, (nq,))
    _check(q, "q", cache.k.dtype, (T, nq * hd))
    _check(out, "out", cache.k.dtype, (T, nq * hd))
    _check_paged(meta, cache, T)
    if tuple(cache.k.shape[1:]) != (nkv, cache.page_size, hd):
        raise BackendError(f"cache pages {list(cache.k.shape)} do not fit {nkv} kv heads of {hd}")
    lib.call("attention_plain", "hb_attention_plain", q.data_ptr(), cache.k.data_ptr(),
             cache.v.data_ptr(), out.data_ptr(), dtype_code(q), meta.positions.data_ptr(),
             meta.seq_of.data_ptr(), meta.slots.data_ptr(), cache.page_table.data_ptr(),
             cache.page_table.shape[1], cache.page_size, T, nq, nkv, hd, float(scale),
             int(window or 0), _ptr(sinks), int(chunk or 0), float(softcap or 0.0), _stream())


GLU_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def swiglu(gu, out, activation="silu"):
    """out[t, i] = f(gu[t, i]) * gu[t, I + i]; gu f32 [T, 2I]; f "silu" or "gelu_tanh"."""
    if activation not in GLU_ACTIVATIONS:
        raise BackendError(f"gated linear unit: unknown activation {activation!r}")
    _check(gu, "gate_up", torch.float32, (None, None))
    T, two_i = gu.shape
    if two_i % 2:
        raise BackendError("swiglu: the input's width must be even")
    _check(out, "out", None, (T, two_i // 2))
    lib.call("elementwise", "hb_swiglu", gu.data_ptr(), out.data_ptr(), dtype_code(out), T, two_i // 2,
             GLU_ACTIVATIONS[activation], _stream())


def fill_u32(t, value):
    """Set every 32-bit word of a tensor (through a kernel, safe inside a captured graph)."""
    _check(t, "tensor")
    nbytes = t.numel() * t.element_size()
    if nbytes % 4:
        raise BackendError("fill: the tensor's size is no multiple of 4 bytes")
    lib.call("elementwise", "hb_fill_u32", t.data_ptr(), int(value), nbytes // 4, _stream())


ARGMAX_MAX_CHUNKS = 64


def argmax_scratch(rows, device):
    """The partial results of the first of argmax's two stages for up to `rows` rows, to be kept
    and handed to `argmax` again and again."""
    return (torch.empty((rows, ARGMAX_MAX_CHUNKS), dtype=torch.float32, device=device),
            torch.empty((rows, ARGMAX_MAX_CHUNKS), dtype=torch.int32, device=device))


def argmax(logits, out, scratch=None):
    """out[r] = first index of the largest value of logits[r]; logits f32 [R, V], out int32 [R].
    `scratch` as `argmax_scratch` makes it (for at least R rows), else it is allocated here."""
    _check(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    _check(out, "out", torch.int32, (R,))
    chunks = max(1, min(ARGMAX_MAX_CHUNKS, V // 8192, 1024 // R if R <= 1024 else 1))
    sv = si = None
    if chunks > 1 and scratch is not None:
        sv, si = scratch
        _check(sv, "argmax scratch values", torch.float32, (None, ARGMAX_MAX_CHUNKS))
        _check(si, "argmax scratch indices", torch.int32, tuple(sv.shape))
        if sv.shape[0] < R:
            raise BackendError("argmax: the scratch has fewer rows than the logits")
    elif chunks > 1:
        sv = torch.empty((R, chunks), dtype=torch.float32, device=logits.device)
        si = torch.empty((R, chunks), dtype=torch.int32, device=logits.device)
    lib.call("sampling", "hb_argmax", logits.data_ptr(), V, R, V, out.data_ptr(), _ptr(sv), _ptr(si),
             chunks, _stream())


SAMPLE_CHUNK = 8192


def sample(logits, temperature, top_k, top_p, rng_states, rng_index, out, scratch=None, sifted=None):
    """One token per row by temperature / top-k / top-p; rng_states int64 [n], advanced in place.

    `scratch` = (keys int32 [R, P2], idx int32 [R, P2]) with P2 the power of two >= V; needed
    unless 0 < top_k <= 1024 and top_k < V.
    `sifted` = (keys int32, idx int32), each of at least R * ceil(V / 8192) * top_k elements, optional:
    with them a long row is first sifted by a block for every 8192 logits (same result, sooner).
    """
    _check(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    _check(out, "out", torch.int32, (R,))
    _check(rng_states, "rng_states", torch.int64, (None,))
    if rng_index is not None:
        _check(rng_index, "rng_index", torch.int32, (R,))
    elif rng_states.shape[0] < R:
        raise BackendError("sample: fewer generator states than rows")
    keys = idx = None
    p2 = 0
    if scratch is not None:
        keys, idx = scratch
        p2 = keys.shape[1]
        _check(keys, "scratch keys", torch.int32, (None, p2))
        _check(idx, "scratch idx", torch.int32, tuple(keys.shape))
        if keys.shape[0] < R:
            raise BackendError("sample: scratch has fewer rows than the logits")
    pre_key = pre_idx = None
    if sifted is not None:
        pre_key, pre_idx = sifted
        need = R * (-(-V // SAMPLE_CHUNK)) * max(int(top_k), 1)
        _check(pre_key, "sifted keys", torch.int32, (None,))
        _check(pre_idx, "sifted idx", torch.int32, (None,))
        if pre_key.numel() < need or pre_idx.numel() < need:
            raise BackendError(f"sample: the buffers for sifted candidates hold fewer than {need} elements")
    lib.call("sampling", "hb_sample", logits.data_ptr(), V, R, V, float(temperature), int(top_k),
             float(top_p), rng_states.data_ptr(), _ptr(rng_index), out.data_ptr(), _ptr(keys),
             _ptr(idx), p2, _ptr(pre_key), _ptr(pre_idx), _stream())


NUCLEUS_CANDIDATES = 1024


def nucleus_buffers(rows, vocab, device):
    """(keys int32, idx int32, sums float32) that sample_nucleus needs for `rows` rows of `vocab` logits."""
    chunks = -(-vocab // SAMPLE_CHUNK)
    return (torch.empty(rows * chunks * NUCLEUS_CANDIDATES, dtype=torch.int32, device=device),
            torch.empty(rows * chunks * NUCLEUS_CANDIDATES, dtype=torch.int32, device=device),
            torch.empty(rows * chunks * 2, dtype=torch.float32, device=device))


def sample_nucleus(logits, temperature, top_p, rng_states, rng_index, out, buffers):
    """Top-p without top-k on rows of more than 1024 logits, the quick way: a row's prefix is looked
    for among its 1024 largest logits only (the softmax still runs over the whole row). A row whose
    prefix does not end among them gets out[r] = -1 and keeps its generator state: sample it with
    `sample`. `buffers` as `nucleus_buffers` makes them."""
    _check(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    _check(out, "out", torch.int32, (R,))
    _check(rng_states, "rng_states", torch.int64, (None,))
    if rng_index is not None:
        _check(rng_index, "rng_index", torch.int32, (R,))
    elif rng_states.shape[0] < R:
        raise BackendError("sample: fewer generator states than rows")
    keys, idx, sums = buffers
    chunks = -(-V // SAMPLE_CHUNK)
    _check(keys, "candidate keys", torch.int32, (None,))
    _check(idx, "candidate idx", torch.int32, (None,))
    _check(sums, "chunk sums", torch.float32, (None,))
    if min(keys.numel(), idx.numel()) < R * chunks * NUCLEUS_CANDIDATES or sums.numel() < R * chunks * 2:
        raise BackendError("sample: the buffers of the quick top-p are too small for these logits")
    lib.call("sampling", "hb_sample_nucleus", logits.data_ptr(), V, R, V, float(temperature), float(top_p),
             rng_states.data_ptr(), _ptr(rng_index), out.data_ptr(), keys.data_ptr(), idx.data_ptr(),
             sums.data_ptr(), _stream())


def sample_all(logits, temperature, rng_states, rng_index, out, sums):
    """Temperature sampling over whole rows (no top-k, no top-p): a block for every 8192 logits adds
    up its part of the softmax, a block a row takes the draw and walks the chunk it falls into.
    `sums`: float32 of at least R * ceil(V / 8192) * 2 elements."""
    _check(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    _check(out, "out", torch.int32, (R,))
    _check(rng_states, "rng_states", torch.int64, (None,))
    if rng_index is not None:
        _check(rng_index, "rng_index", torch.int32, (R,))
    elif rng_states.shape[0] < R:
        raise BackendError("sample: fewer generator states than rows")
    _check(sums, "chunk sums", torch.float32, (None,))
    if sums.numel() < R * (-(-V // SAMPLE_CHUNK)) * 2:
        raise BackendError("sample: the buffer of the chunks' sums is too small for these logits")
    lib.call("sampling", "hb_sample_all", logits.data_ptr(), V, R, V, float(temperature), rng_states.data_ptr(),
             _ptr(rng_index), out.data_ptr(), sums.data_ptr(), _stream())


def force_tokens(logits, rows, tokens):
    """Every logit of row rows[i] but that of tokens[i] becomes -inf, in place: the next choice in
    that row can only be that token. rows, tokens: lists of ints (checked here against the shape)."""
    _check(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    if len(rows) != len(tokens) or not rows:
        raise BackendError("force_tokens: needs as many tokens as rows, at least one")
    for r, t in zip(rows, tokens):
        if not (0 <= int(r) < R and 0 <= int(t) < V):
            raise BackendError(f"force_tokens: row {r} or token {t} outside logits of shape {R} x {V}")
    both = torch.tensor([list(map(int, rows)), list(map(int, tokens))], dtype=torch.int32, device=logits.device)
    lib.call("sampling", "hb_force_tokens", logits.data_ptr(), V, R, V, both[0].data_ptr(), both[1].data_ptr(),
             len(rows), _stream())


def layernorm(x, weight, out, eps, rows=None, delta=None, mult=1.0):
    """out[r] = (x[r] - mean) / sqrt(var + eps) * weight, var the mean of the squared deviations; x f32
    [T, H] (rows int32: only these, gathered), out f32 or the compute dtype, and it may be x itself.
    delta f32 [T, H]: x becomes x + mult * delta first, in place, and that sum is normed (no rows then);
    out None with a delta: only the sum."""
    _check(x, "x", torch.float32, (None, None))
    H = x.shape[1]
    _check(weight, "weight", torch.float32, (H,))
    if rows is not None:
        _check(rows, "rows", torch.int32, (None,))
        R = rows.shape[0]
    else:
        R = x.shape[0]
    if delta is not None:
        _check(delta, "delta", torch.float32, tuple(x.shape))
        if rows is not None:
            raise BackendError("layernorm: rows are not gathered while a sum is added")
    elif out is None:
        raise BackendError("layernorm: nothing to do")
    if out is not None:
        _check(out, "out", None, (R, H))
    lib.call("elementwise", "hb_layernorm", x.data_ptr(), _ptr(delta), float(mult), weight.data_ptr(), _ptr(out),
             dtype_code(out) if out is not None else F32, _ptr(rows), R, H, float(eps), _stream())


def scale(x, factor):
    """x *= factor in place; x float32."""
    _check(x, "x", torch.float32)
    lib.call("elementwise", "hb_scale", x.data_ptr(), float(factor), x.numel(), _stream())


def gemm_plain_batched(a, w, c, M, N, K, lda, ldw, ldc, batch, batch_a, batch_w, batch_c):
    """`batch` products c_b[M, N] = a_b[M, K] @ w_b[N, K]^T in one launch, float32 arithmetic: product b
    reads a + b * batch_a, w + b * batch_w and writes c + b * batch_c (elements), rows lda / ldw / ldc
    elements apart. The caller's tensors must hold every element that this addresses."""
    for t, name, ld, rows, cols, step in ((a, "a", lda, M, K, batch_a), (w, "w", ldw, N, K, batch_w),
                                          (c, "c", ldc, M, N, batch_c)):
        _check(t, name)
        last = (batch - 1) * step + (rows - 1) * ld + cols
        if ld < cols or last > t.numel():
            raise BackendError(f"batched gemm: {name} of {t.numel()} elements does not hold the batch (needs {last})")
    lib.call("gemm_plain", "hb_gemm_plain_batched", a.data_ptr(), dtype_code(a), w.data_ptr(), dtype_code(w),
             c.data_ptr(), dtype_code(c), M, N, K, lda, ldw, ldc, batch, batch_a, batch_w, batch_c, _stream())


def layernorm_free_sum(x, delta, mult):
    """x += mult * delta, float32 in place (the layer norm's kernel without its norm)."""
    _check(x, "x", torch.float32, (None, None))
    _check(delta, "delta", torch.float32, tuple(x.shape))
    lib.call("elementwise", "hb_layernorm", x.data_ptr(), delta.data_ptr(), float(mult), None, None, F32, None,
             x.shape[0], x.shape[1], 0.0, _stream())


def postnorm(src, weight, x, y, eps, alpha_next, acc=None):
    """Between two parts of a layer whose norm comes after the sum: x = src / rms(src) * weight (weight
    None: x = src), y = x in y's dtype, acc = alpha_next * x (alpha_next 0: none). src f32 [T, H]; x f32
    [T, H] or None; y [T, H] or None; acc f32 [T, H], src itself if not given."""
    _check(src, "src", torch.float32, (None, None))
    T, H = src.shape
    if acc is None:
        acc = src
    else:
        _check(acc, "acc", torch.float32, (T, H))
    if weight is not None:
        _check(weight, "weight", torch.float32, (H,))
    for t, name in ((x, "x"), (y, "y")):
        if t is not None:
            _check(t, name, torch.float32 if name == "x" else None, (T, H))
            if t.data_ptr() in (src.data_ptr(), acc.data_ptr()):
                raise BackendError(f"postnorm: {name} must be other rows than the source and the sum")
    lib.call("elementwise", "hb_postnorm", src.data_ptr(), _ptr(weight), _ptr(x), _ptr(y),
             dtype_code(y) if y is not None else F32, acc.data_ptr(), T, H, float(eps), float(alpha_next),
             _stream())


def relu_squared(z, out):
    """out = max(z, 0)^2; z f32, out of the same shape in any storage type."""
    _check(z, "z", torch.float32)
    _check(out, "out", None, tuple(z.shape))
    lib.call("elementwise", "hb_relu_squared", z.data_ptr(), out.data_ptr(), dtype_code(out), z.numel(), _stream())


def gemm_plain_columns(a, col0, K, w, c, accumulate=False, decay=None):
    """c[M, N] (+)= a[:, col0:col0 + K] @ w[N, K]^T in float32 arithmetic: the product of some columns of
    wider rows, read where they lie. (Up to 32 float32 rows times bfloat16 rows, k in steps of 32: a kernel of
    more and smaller workgroups than the tiled one, which a short k leaves with few.)
    decay (a_log f32 [N / D], dt_bias f32 [N], D): the sums are a decay's pre-activations, and c (float32, not
    added to) takes the decays themselves, exp(-exp(a_log[n // D]) softplus(sum + dt_bias[n])), as
    `recurrent.channel_decay` makes them from rows in memory.
    decay ("sigmoid_root", bias f32 [N], root): c takes sigmoid(sum + bias[n])^root instead."""
    _check(a, "a", None, (None, None))
    _check(w, "w", None, (None, K))
    M, lda = a.shape
    N = w.shape[0]
    if col0 < 0 or col0 + K > lda:
        raise BackendError(f"gemm: columns [{col0}, {col0 + K}) of rows of {lda}")
    _check(c, "c", None, (M, N))
    if accumulate and c.dtype != torch.float32:
        raise BackendError("gemm: accumulation needs a float32 output")
    a_log = dt_bias = D = 0
    root = 0.0
    if decay is not None and decay[0] == "sigmoid_root":
        _, bias, root = decay
        if accumulate or c.dtype != torch.float32:
            raise BackendError("gemm: a decay is float32, stored and not added to")
        _check(bias, "decay bias", torch.float32, (N,))
        a_log = dt_bias = bias.data_ptr()
        D = 1
    elif decay is not None:
        rate, bias, D = decay
        if accumulate or c.dtype != torch.float32 or D <= 0 or N % D:
            raise BackendError("gemm: a decay is float32, stored and not added to, its columns whole heads")
        _check(rate, "A_log", torch.float32, (N // D,))
        _check(bias, "dt_bias", torch.float32, (N,))
        a_log, dt_bias = rate.data_ptr(), bias.data_ptr()
    lib.call("gemm_plain", "hb_gemm_plain_short_k", a.data_ptr() + col0 * a.element_size(), dtype_code(a), w.data_ptr(),
             dtype_code(w), c.data_ptr(), dtype_code(c), M, N, K, lda, K, N, 1 if accumulate else 0, a_log, dt_bias,
             int(D), float(root), _stream())


def rmsnorm_scaled_sum(x, delta, factors, weight, out, eps):
    """x += factors * delta (a factor a column), in place, then out = x / rms(x) * weight; x, delta f32 [T, H],
    factors f32 [H]. out None (weight may then be None): only the sum."""
    _check(x, "x", torch.float32, (None, None))
    T, H = x.shape
    _check(delta, "delta", torch.float32, (T, H))
    _check(factors, "factors", torch.float32, (H,))
    if out is not None:
        _check(weight, "weight", torch.float32, (H,))
        _check(out, "out", None, (T, H))
        if out.data_ptr() in (x.data_ptr(), delta.data_ptr()):
            raise BackendError("rmsnorm: the normed rows must be other rows than the sum's")
    lib.call("elementwise", "hb_rmsnorm_scaled_sum", x.data_ptr(), delta.data_ptr(), factors.data_ptr(), _ptr(weight),
             _ptr(out), dtype_code(out) if out is not None else F32, T, H, float(eps), _stream())


def normed_pair(a, wa, ca, b, wb, cb, out, eps, accumulate=False):
    """out (+)= ca * a / rms(a) * wa + cb * b / rms(b) * wb, row by row; all f32 [T, H], weights [H]."""
    _check(a, "a", torch.float32, (None, None))
    T, H = a.shape
    _check(b, "b", torch.float32, (T, H))
    _check(out, "out", torch.float32, (T, H))
    _check(wa, "wa", torch.float32, (H,))
    _check(wb, "wb", torch.float32, (H,))
    lib.call("elementwise", "hb_normed_pair", a.data_ptr(), wa.data_ptr(), float(ca), b.data_ptr(), wb.data_ptr(), float(cb),
             out.data_ptr(), T, H, float(eps), 1 if accumulate else 0, _stream())


def filter_norm_rotate_write(proj, taps, filter_state, q_norm_w, k_norm_w, rates, rot_dims, meta, cache, q_out,
                             nq, nkv, dim, vdim, hd, eps, bias=None, head_norm=False):
    """The first columns of proj's rows (f32 [T, ld]) are [nq x dim queries | nkv x dim keys | nkv x vdim values]:
    filtered along time (taps f32 [C, K] with the slot's last inputs in filter_state f32 [slots, K - 1, C]; None:
    no filter), queries and keys each normed over the whole projection (weights [nq x dim], [nkv x dim]; None:
    no norm), neighbouring pairs of the first rot_dims entries of every head turned by position x rates (f64
    [rot_dims / 2]; None: no rotation); q to q_out [T, nq x hd], keys and values to the token's page, heads kept
    at hd with zeros beyond their own size. The filter's state is moved on too: by the kernel itself where every
    sequence brings one token (meta.max_new), by the filter-state kernel afterwards otherwise.
    bias f32 [C]: added to the channels after the filter. head_norm: every query head and every key head is
    normed by itself, with weights [dim] that all heads share."""
    T, ld = proj.shape
    C = (nq + nkv) * dim + nkv * vdim
    _check(proj, "proj", torch.float32, (T, ld))
    K = 0
    if taps is not None:
        K = taps.shape[1]
        _check(taps, "taps", torch.float32, (C, K))
        if K > 1:
            _check(filter_state, "filter_state", torch.float32, (None, K - 1, C))
    if head_norm and (q_norm_w is None or k_norm_w is None):
        raise BackendError("filtered attention: a norm a head needs its weights")
    if q_norm_w is not None:
        _check(q_norm_w, "q_norm", torch.float32, (dim if head_norm else nq * dim,))
    if k_norm_w is not None:
        _check(k_norm_w, "k_norm", torch.float32, (dim if head_norm else nkv * dim,))
    if bias is not None:
        _check(bias, "bias", torch.float32, (C,))
    if rates is not None:
        _check(rates, "rates", torch.float64, (rot_dims // 2,))
    _check_paged(meta, cache, T)
    _check(meta.seq_starts, "seq_starts", torch.int32, (meta.num_seqs + 1,))
    _check(q_out, "q_out", cache.k.dtype, (T, nq * hd))
    if tuple(cache.k.shape[1:]) != (nkv, cache.page_size, hd):
        raise BackendError(f"cache pages {list(cache.k.shape)} do not fit {nkv} kv heads of {hd}")
    if ld < C or hd < max(dim, vdim):
        raise BackendError(f"filtered attention: rows of {ld} for {C} channels, heads of {dim} and {vdim} kept at {hd}")
    lib.call("elementwise", "hb_filter_norm_rotate_write", proj.data_ptr(), ld, _ptr(taps), K,
             _ptr(filter_state) if K > 1 else None, _ptr(q_norm_w), _ptr(k_norm_w), _ptr(rates), int(rot_dims),
             meta.positions.data_ptr(), meta.seq_of.data_ptr(), meta.seq_starts.data_ptr(), meta.slots.data_ptr(),
             cache.page_table.data_ptr(), cache.page_table.shape[1], cache.page_size, q_out.data_ptr(),
             cache.k.data_ptr(), cache.v.data_ptr(), dtype_code(q_out), T, nq, nkv, dim, vdim, hd, float(eps),
             int(meta.max_new), _ptr(bias), 1 if head_norm else 0, _stream())
    if K > 1 and meta.max_new != 1:
        _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
        lib.call("recurrent", "hb_filter_state", proj.data_ptr(), ld, filter_state.data_ptr(), meta.seq_starts.data_ptr(),
                 meta.slots.data_ptr(), meta.num_seqs, C, K, None, _stream())


def add_bias(x, bias):
    """x[t, :] += bias: x f32 [T, H], bias f32 [H]."""
    T, H = x.shape
    _check(x, "x", torch.float32, (T, H))
    _check(bias, "bias", torch.float32, (H,))
    lib.call("elementwise", "hb_add_bias", x.data_ptr(), bias.data_ptr(), T, H, _stream())


TOKEN_SIDE_FEW = 64      # up to so many tokens the gate's rows take a workgroup each


def token_side(x, token_ids, table, col0, w_gate, w_proj_t, norm_w, eps, g, y, stage=1, g16=None):
    """x += rmsnorm(W_proj (gelu_tanh(W_gate x) * table[token, col0 : col0 + D])) * norm_w, row by row and in
    place: x f32 [T, H], token_ids int32 [T], table [V, ld], W_gate [D, H], W_proj transposed [D, H] (one dtype),
    norm_w f32 [H]; g f32 [T, D] and y f32 [T, H] are scratch. stage 0: the gate alone (more than TOKEN_SIDE_FEW
    tokens: into g16 bf16 [T, D] if that is given, for a product of the caller's that makes y); stage 2: the norm
    and the sum alone, from y."""
    if g16 is not None:
        _check(g16, "g16", torch.bfloat16, (x.shape[0], w_gate.shape[0]))
        if stage != 0 or x.shape[0] <= TOKEN_SIDE_FEW:
            raise BackendError("token input: bfloat16 gates are for many tokens and a product of the caller's")
    T, H = x.shape
    D = w_gate.shape[0]
    _check(x, "x", torch.float32, (T, H))
    _check(token_ids, "token_ids", torch.int32, (T,))
    _check(table, "table", w_gate.dtype, (None, None))
    _check(w_gate, "gate", None, (D, H))
    _check(w_proj_t, "proj (transposed)", w_gate.dtype, (D, H))
    _check(norm_w, "norm", torch.float32, (H,))
    _check(g, "g", torch.float32, (T, D))
    _check(y, "y", torch.float32, (T, H))
    if col0 < 0 or col0 + D > table.shape[1]:
        raise BackendError("token input: the layer's columns lie outside the table's rows")
    lib.call("elementwise", "hb_token_side", x.data_ptr(), token_ids.data_ptr(), table.data_ptr(), table.shape[1],
             int(col0), w_gate.data_ptr(), w_proj_t.data_ptr(), dtype_code(w_gate), norm_w.data_ptr(), g.data_ptr(),
             _ptr(g16), y.data_ptr(), T, H, D, float(eps), int(stage), _stream())


def gate_heads(attn, gate_rows, g_off, out, nq, hd, vdim):
    """out[t, h vdim + d] = attn[t, h hd + d] * sigmoid(gate_rows[t, g_off + h vdim + d]), d < vdim; attn [T, nq hd]
    and out [T, nq vdim] of one dtype, gate_rows f32 [T, ld] (None: no gate, the heads only leave at their own size)."""
    T = attn.shape[0]
    _check(attn, "attn", None, (T, nq * hd))
    _check(out, "out", attn.dtype, (T, nq * vdim))
    ld = 0
    if gate_rows is not None:
        _check(gate_rows, "gate", torch.float32, (T, None))
        ld = gate_rows.shape[1]
        if g_off < 0 or g_off + nq * vdim > ld:
            raise BackendError("gate: its columns lie outside the rows")
    lib.call("elementwise", "hb_gate_heads", attn.data_ptr(), dtype_code(attn), _ptr(gate_rows), ld, int(g_off),
             out.data_ptr(), T, nq, hd, vdim, _stream())
