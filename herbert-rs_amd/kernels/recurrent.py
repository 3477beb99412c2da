"""Host side of the kernels for mixers with state of fixed size (csrc/recurrent.hip): the short
causal convolution with its activation and unit vectors, the gated delta rule, and the gated norm a
head that follows it. Operand checks, then the launch."""
import torch

from ..errors import BackendError
from . import lib
from .ops import _check, _stream, dtype_code

MAX_TAPS = 16
MAX_KEY_DIM = 256


def conv_silu(proj, taps, conv_state, meta, out, n_unit, unit_dim, n_scaled, scale, unit_eps, n_plain, plain_dim,
              col0=0, bias=None):
    """out[t, c] = silu(sum_j taps[c, j] * input[t - (K - 1) + j, c]) over the C columns of proj (f32 [T, ld])
    from col0 on; inputs from before the step come from conv_state (f32 [slots, K - 1, C]), which is
    then moved on. The first n_unit sections of unit_dim channels become unit vectors (the first
    n_scaled of them times `scale`), the n_plain sections of plain_dim that follow stay as they are (the last
    of them may be shorter). bias f32 [C]: the sums start there."""
    T, ld = proj.shape
    C, K = taps.shape
    if bias is not None:
        _check(bias, "conv bias", torch.float32, (C,))
    _check(proj, "proj", torch.float32, (T, ld))
    _check(taps, "taps", torch.float32, (C, K))
    _check(conv_state, "conv_state", torch.float32, (None, max(K - 1, 1), C))
    _check(out, "out", torch.float32, (T, C))
    _check(meta.seq_of, "seq_of", torch.int32, (T,))
    _check(meta.seq_starts, "seq_starts", torch.int32, (meta.num_seqs + 1,))
    _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
    if n_unit * unit_dim + n_plain * plain_dim < C or col0 < 0 or ld < col0 + C or not 1 <= K <= MAX_TAPS:
        raise BackendError(f"conv: sections {n_unit} x {unit_dim} + {n_plain} x {plain_dim} do not fit {C} channels "
                           f"of {K} taps")
    lib.call("recurrent", "hb_conv_silu", proj.data_ptr() + 4 * col0, ld, taps.data_ptr(), conv_state.data_ptr(),
             meta.seq_of.data_ptr(), meta.seq_starts.data_ptr(), meta.slots.data_ptr(), out.data_ptr(), T,
             meta.num_seqs, C, K, n_unit, unit_dim, n_scaled, float(scale), float(unit_eps), n_plain, plain_dim,
             None if bias is None else bias.data_ptr(), _stream())


MAX_SSM_STATE = 256


def ssm_state_floats(N, P):
    """Floats of state that the walk's kernel keeps for a head of N rows and P columns (its own layout: every
    thread's numbers side by side, rows and columns rounded up to what its lanes hold). The kernel's entry point
    refuses a state of another size, so the two cannot drift apart unseen."""
    if not 0 < N <= MAX_SSM_STATE or P <= 0:
        raise BackendError(f"state-space walk: a state of {N} x {P}")
    nr, lpc = (4, 4) if N <= 16 else (4, 8) if N <= 32 else (4, 16) if N <= 64 else (8, 16) if N <= 128 else (16, 16)
    cols = 256 // lpc
    return -(-P // cols) * 256 * nr


def ssm_scan(u, proj, dt_off, dt_bias, a_log, d_skip, state, meta, out, heads, groups, N, P):
    """The state-space walk of every sequence of the step: u f32 [T, heads P + 2 groups N] (x, B, C as the
    convolution left them), the step sizes' pre-activations in columns [dt_off, + heads) of proj (f32 [T, ld]);
    dt = softplus(. + dt_bias), S <- exp(-exp(a_log) dt) S + dt B x^T, out = S^T C + d_skip x; state f32
    [slots, heads, ssm_state_floats(N, P)] advanced in place (zeros: an empty state), out f32 [T, heads P]."""
    T = u.shape[0]
    _check(u, "u", torch.float32, (T, heads * P + 2 * groups * N))
    _check(proj, "proj", torch.float32, (T, None))
    for t, name in ((dt_bias, "dt_bias"), (a_log, "A_log"), (d_skip, "D")):
        _check(t, name, torch.float32, (heads,))
    _check(state, "state", torch.float32, (None, heads, ssm_state_floats(N, P)))
    _check(out, "out", torch.float32, (T, heads * P))
    _check(meta.seq_starts, "seq_starts", torch.int32, (meta.num_seqs + 1,))
    _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
    if heads % groups or not 0 < N <= MAX_SSM_STATE or dt_off < 0 or dt_off + heads > proj.shape[1]:
        raise BackendError(f"state-space walk: {heads} heads in {groups} groups, a state of {N} rows")
    lib.call("recurrent", "hb_ssm_scan", u.data_ptr(), u.shape[1], proj.data_ptr(), proj.shape[1], int(dt_off),
             dt_bias.data_ptr(), a_log.data_ptr(), d_skip.data_ptr(), state.data_ptr(), meta.seq_starts.data_ptr(),
             meta.slots.data_ptr(), out.data_ptr(), meta.num_seqs, heads, groups, N, P, state.shape[2], _stream())


def gated_group_norm(o, proj, z_off, weight, out, parts, eps):
    """out = v / rms(v) * weight with v = o * silu(proj[:, z_off ...]), the root mean square taken over each of
    `parts` equal groups of a row by itself; o f32 [T, width], weight f32 [width], out in any dtype."""
    T, width = o.shape
    _check(o, "o", torch.float32, (T, width))
    _check(proj, "proj", torch.float32, (T, None))
    _check(weight, "weight", torch.float32, (width,))
    _check(out, "out", None, (T, width))
    if parts <= 0 or width % parts or z_off < 0 or z_off + width > proj.shape[1]:
        raise BackendError(f"gated norm in groups: {width} columns in {parts} groups")
    lib.call("recurrent", "hb_gated_group_norm", o.data_ptr(), proj.data_ptr(), proj.shape[1], int(z_off),
             weight.data_ptr(), out.data_ptr(), dtype_code(out), T, width, int(parts), float(eps), _stream())


def gated_delta(qkv, proj, b_off, a_off, a_log, dt_bias, state, meta, out, kv_heads, heads, D, V, decay=None,
                correction=True, out_scale=1.0):
    """The delta rule over every sequence of the step; qkv f32 [T, at least 2 kv_heads D + heads V] (queries,
    keys, values in a row's first columns), proj f32 [T, ld] with column b_off + h (beta's pre-activation) and a_off + h (the
    decay's), state f32 [slots, heads, D, V] advanced in place, out f32 [T, heads V].
    decay f32 [T, heads D]: a factor a key channel, as `channel_decay` leaves it; a_off, a_log and
    dt_bias are then not read (they may be None). correction False (a decay a key channel must be given):
    the linear attention S <- diag(decay) S + k v^T, o = S^T q; proj is then not read (it may be None).
    out_scale: o is multiplied by it."""
    T, C = qkv.shape
    if not correction:
        if decay is None:
            raise BackendError("linear attention: the walk without a correction takes a decay a key channel")
        _check(decay, "decay", torch.float32, (T, heads * D))
        _check(qkv, "qkv", torch.float32, (T, None))
        _check(state, "state", torch.float32, (None, heads, D, V))
        _check(out, "out", torch.float32, (T, heads * V))
        _check(meta.seq_starts, "seq_starts", torch.int32, (meta.num_seqs + 1,))
        _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
        if heads % kv_heads or not 0 < D <= MAX_KEY_DIM or C < 2 * kv_heads * D + heads * V:
            raise BackendError(f"linear attention: {heads} heads on {kv_heads} key heads of {D} in rows of {C}")
        lib.call("recurrent", "hb_gated_delta", qkv.data_ptr(), C, None, 0, 0, 0, None, None, decay.data_ptr(),
                 state.data_ptr(), meta.seq_starts.data_ptr(), meta.slots.data_ptr(), out.data_ptr(), meta.num_seqs,
                 kv_heads, heads, D, V, 0, float(out_scale), _stream())
        return
    if decay is not None:
        _check(decay, "decay", torch.float32, (T, heads * D))
        a_off = 0
    else:
        _check(a_log, "A_log", torch.float32, (heads,))
        _check(dt_bias, "dt_bias", torch.float32, (heads,))
    _check(qkv, "qkv", torch.float32, (T, 2 * kv_heads * D + heads * V))
    _check(proj, "proj", torch.float32, (T, None))
    ld = proj.shape[1]
    if not (0 <= b_off and b_off + heads <= ld and 0 <= a_off and a_off + heads <= ld):
        raise BackendError("delta rule: the gate columns lie outside the projection's rows")
    _check(state, "state", torch.float32, (None, heads, D, V))
    _check(out, "out", torch.float32, (T, heads * V))
    _check(meta.seq_starts, "seq_starts", torch.int32, (meta.num_seqs + 1,))
    _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
    if heads % kv_heads or not 0 < D <= MAX_KEY_DIM:
        raise BackendError(f"delta rule: {heads} heads on {kv_heads} key heads of {D}")
    lib.call("recurrent", "hb_gated_delta", qkv.data_ptr(), C, proj.data_ptr(), ld, b_off, a_off,
             None if decay is not None else a_log.data_ptr(), None if decay is not None else dt_bias.data_ptr(),
             None if decay is None else decay.data_ptr(), state.data_ptr(), meta.seq_starts.data_ptr(),
             meta.slots.data_ptr(),
             out.data_ptr(), meta.num_seqs, kv_heads, heads, D, V, 1, float(out_scale), _stream())


def gated_head_norm(o, proj, g_off, weight, out, heads, V, eps, gate="silu"):
    """out[t, h, :] = o[t, h, :] / rms * weight * gate(proj[t, g_off + h V ...]), gate "silu" or
    "sigmoid"; out in any dtype."""
    if gate not in ("silu", "sigmoid"):
        raise BackendError(f"gated norm: unknown gate {gate!r}")
    T = o.shape[0]
    _check(o, "o", torch.float32, (T, heads * V))
    _check(proj, "proj", torch.float32, (T, None))
    if g_off < 0 or g_off + heads * V > proj.shape[1]:
        raise BackendError("gated norm: the gate columns lie outside the projection's rows")
    _check(weight, "weight", torch.float32, (V,))
    _check(out, "out", None, (T, heads * V))
    lib.call("recurrent", "hb_gated_head_norm", o.data_ptr(), proj.data_ptr(), proj.shape[1], g_off, weight.data_ptr(),
             out.data_ptr(), dtype_code(out), T, heads, V, float(eps), 1 if gate == "sigmoid" else 0, _stream())


def channel_decay(z, z_off, a_log, dt_bias, out, heads, D):
    """out[t, h, d] = exp(-exp(a_log[h]) * softplus(z[t, z_off + h D + d] + dt_bias[h, d])): the delta rule's
    decay a key channel from its pre-activation. z f32 [T, ld]; out f32 [T, heads D], which may be z
    itself (z_off 0, ld = heads D)."""
    T, ld = z.shape
    _check(z, "z", torch.float32, (T, ld))
    _check(out, "out", torch.float32, (T, heads * D))
    _check(a_log, "A_log", torch.float32, (heads,))
    _check(dt_bias, "dt_bias", torch.float32, (heads * D,))
    if z_off < 0 or z_off + heads * D > ld or (out.data_ptr() == z.data_ptr() and (z_off or ld != heads * D)):
        raise BackendError("channel decay: the pre-activations lie outside their rows")
    lib.call("recurrent", "hb_channel_decay", z.data_ptr() + 4 * z_off, ld, a_log.data_ptr(), dt_bias.data_ptr(),
             out.data_ptr(), T, heads, D, _stream())


def filter_state(proj, conv_state, meta, C, K, bias=None):
    """After a step: conv_state (f32 [slots, K - 1, C]) takes the last K - 1 inputs of each sequence, the first C
    columns of proj's rows (f32 [T, ld]) plus bias (f32 [C]) if given. For mixers that filter in a kernel of
    their own."""
    T, ld = proj.shape
    _check(proj, "proj", torch.float32, (T, ld))
    if K <= 1:
        return
    _check(conv_state, "conv_state", torch.float32, (None, K - 1, C))
    _check(meta.seq_starts, "seq_starts", torch.int32, (meta.num_seqs + 1,))
    _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
    if bias is not None:
        _check(bias, "bias", torch.float32, (C,))
    if ld < C or K > MAX_TAPS:
        raise BackendError(f"filter state: {C} channels of {K} taps in rows of {ld}")
    lib.call("recurrent", "hb_filter_state", proj.data_ptr(), ld, conv_state.data_ptr(), meta.seq_starts.data_ptr(),
             meta.slots.data_ptr(), meta.num_seqs, C, K, None if bias is None else bias.data_ptr(), _stream())


def lru_inputs(proj, bx, by, taps, filter_bias, conv_state, meta, out):
    """The two branches of a gated linear recurrent unit from the projection's rows [x | y] (f32 [T, ld], W
    channels each): out f32 [T, 2 W] = [filter(x + bx) + filter_bias | gelu_tanh(y + by)]; taps f32 [W, K],
    conv_state f32 [slots, K - 1, W] (the inputs with their bias), moved on afterwards."""
    T, ld = proj.shape
    W, K = taps.shape
    _check(proj, "proj", torch.float32, (T, ld))
    _check(taps, "taps", torch.float32, (W, K))
    for t, name in ((bx, "x bias"), (by, "y bias")):
        _check(t, name, torch.float32, (W,))
    if filter_bias is not None:
        _check(filter_bias, "filter bias", torch.float32, (W,))
    _check(conv_state, "conv_state", torch.float32, (None, max(K - 1, 1), W))
    _check(out, "out", torch.float32, (T, 2 * W))
    _check(meta.seq_of, "seq_of", torch.int32, (T,))
    _check(meta.seq_starts, "seq_starts", torch.int32, (meta.num_seqs + 1,))
    _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
    if ld < 2 * W or not 1 <= K <= MAX_TAPS:
        raise BackendError(f"recurrent unit: rows of {ld} for 2 x {W} channels, {K} taps")
    lib.call("recurrent", "hb_lru_inputs", proj.data_ptr(), ld, bx.data_ptr(), by.data_ptr(), taps.data_ptr(),
             None if filter_bias is None else filter_bias.data_ptr(), conv_state.data_ptr(), meta.seq_of.data_ptr(),
             meta.seq_starts.data_ptr(), meta.slots.data_ptr(), out.data_ptr(), T, meta.num_seqs, W, K, int(meta.max_new),
             _stream())


def lru_scan(ug, gates, r_bias, i_bias, lam, rate, state, meta, out, block):
    """The recurrence of every sequence of the step, channel by channel: with r = sigmoid(r_pre + r_bias),
    i = sigmoid(i_pre + i_bias), a = exp(-rate r softplus(lam)): S <- a S + sqrt(1 - a^2) i u, out = S g, where
    ug f32 [T, 2 W] = [u | g] and gates f32 [T, 2 W] holds, for every block of `block` channels, that block's
    r_pre then its i_pre; state f32 [slots, W] advanced in place; out [T, W] in any dtype. Where a sequence brings
    128 tokens or more (meta.max_new) a kernel first turns `gates` into decays and inputs where they lie (gates is
    overwritten), and the walk is cut into runs that are walked side by side and joined, which differs from the one
    walk by float32 rounding."""
    T, W2 = ug.shape
    W = W2 // 2
    _check(ug, "ug", torch.float32, (T, 2 * W))
    _check(gates, "gates", torch.float32, (T, 2 * W))
    for t, name in ((r_bias, "r bias"), (i_bias, "i bias"), (lam, "lam")):
        _check(t, name, torch.float32, (W,))
    _check(state, "state", torch.float32, (None, W))
    _check(out, "out", None, (T, W))
    _check(meta.seq_starts, "seq_starts", torch.int32, (meta.num_seqs + 1,))
    _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
    lib.call("recurrent", "hb_lru_scan", ug.data_ptr(), gates.data_ptr(), r_bias.data_ptr(), i_bias.data_ptr(),
             lam.data_ptr(), float(rate), state.data_ptr(), meta.seq_starts.data_ptr(), meta.slots.data_ptr(),
             out.data_ptr(), dtype_code(out), meta.num_seqs, T, W, int(block), int(meta.max_new), _stream())
