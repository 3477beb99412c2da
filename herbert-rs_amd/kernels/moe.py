"""Host side of the routed feed-forward's kernels (csrc/moe.hip): routing and grouping, the products
of an expert's rows with its matrices, the activation, and the weighted sum."""
import torch

from ..errors import BackendError
from . import lib
from .ops import _check, _ptr, _stream, dtype_code

TILE_M = 64
MAX_EXPERTS = 1024


def max_tiles(pairs, experts):
    """The length of the list of row tiles for that many (token, expert) pairs."""
    return (pairs + TILE_M - 1) // TILE_M + experts


class Routing:
    """The buffers that routing fills for a step of T tokens: chosen int32 [T, top], weight f32 [T, top],
    order / row_of int32 [T top], the tiles' lists."""

    def __init__(self, ints, weight, T, E, top, real=None):
        """real: the first `real` of the E experts have matrices (None: all); the others' output is their input."""
        self.real = E if real is None else int(real)
        A, tiles = T * top, max_tiles(T * top, E)
        need = 3 * A + E + 3 * tiles
        if ints.numel() < need or ints.dtype != torch.int32:
            raise BackendError("routing: the int32 buffer is too small")
        self.T, self.E, self.top, self.tiles = T, E, top, tiles
        o = 0
        self.chosen, o = ints[o:o + A], o + A
        self.order, o = ints[o:o + A], o + A
        self.row_of, o = ints[o:o + A], o + A
        self.counts, o = ints[o:o + E], o + E
        self.tile_expert, o = ints[o:o + tiles], o + tiles
        self.tile_row0, o = ints[o:o + tiles], o + tiles
        self.tile_rows, o = ints[o:o + tiles], o + tiles
        self.weight = weight

    @staticmethod
    def ints_needed(T, E, top):
        return 3 * T * top + E + 3 * max_tiles(T * top, E)


def route(logits, bias, routing, scores=False, groups=1, keep=1, score="sigmoid", worth_top=2, renorm=True):
    """logits f32 [T, E] (+ bias f32 [E]) -> routing (see Routing): the largest logits + bias, weighed by a
    softmax over the chosen. The logits' rows may be wider than E (their first E columns count).
    scores=True: s = sigmoid(logit), the choice runs on s + bias within the `keep` best of `groups` equal
    runs of adjacent experts (a group is worth its top two selection values), and the weights are the chosen
    experts' s over their sum. score="softmax": s is the softmax of the logits over all experts; worth_top 1: a
    group is worth its highest selection value alone; renorm False: the weights are the chosen experts' s as they are.
    Experts from routing.real on have no matrices: their pairs' tiles are marked as holding nothing."""
    r = routing
    if score not in ("sigmoid", "softmax") or worth_top not in (1, 2):
        raise BackendError(f"routing: scores are 'sigmoid' or 'softmax', a group is worth its top 1 or 2, not {score!r}, {worth_top}")
    if not 0 < r.real <= r.E:
        raise BackendError(f"routing: {r.real} of {r.E} experts have matrices")
    _check(logits, "logits", torch.float32, (r.T, None))
    ld = logits.shape[1]
    if ld < r.E:
        raise BackendError(f"routing: logits of {ld} columns for {r.E} experts")
    if scores and (groups <= 0 or r.E % groups or not 0 < keep <= groups
                   or r.top > keep * (r.E // groups)):
        raise BackendError(f"routing: {r.top} experts out of {keep} of {groups} groups of {r.E} experts")
    if bias is not None:
        _check(bias, "bias", torch.float32, (r.E,))
    _check(r.weight, "weight", torch.float32, (r.T, r.top))
    if r.E > MAX_EXPERTS or not 0 < r.top <= r.E:
        raise BackendError(f"routing: {r.top} of {r.E} experts")
    lib.call("moe", "hb_moe_route", logits.data_ptr(), _ptr(bias), r.chosen.data_ptr(), r.weight.data_ptr(),
             r.counts.data_ptr(), r.order.data_ptr(), r.row_of.data_ptr(), r.tile_expert.data_ptr(),
             r.tile_row0.data_ptr(), r.tile_rows.data_ptr(), r.T, r.E, r.top, r.tiles, ld, 1 if scores else 0,
             int(groups), int(keep), r.real, 1 if score == "softmax" else 0, int(worth_top), 1 if renorm else 0, _stream())


def gemm_plain(a, w, c, routing, gather):
    """c[row] = a[src(row)] @ w[expert of row]^T for every pair's row; w [E, N, K]; a [T, K] with
    gather (src = the pair's token) or [pairs, K]; c f32 [pairs, N]."""
    r = routing
    E, N, K = w.shape
    _check(w, "w", None, (r.real, N, K))
    _check(a, "a", None, (r.T if gather else r.T * r.top, K))
    _check(c, "c", torch.float32, (r.T * r.top, N))
    lib.call("moe", "hb_moe_gemm_plain", a.data_ptr(), dtype_code(a), w.data_ptr(), dtype_code(w), c.data_ptr(),
             dtype_code(c), r.order.data_ptr(), r.tile_expert.data_ptr(), r.tile_row0.data_ptr(),
             r.tile_rows.data_ptr(), r.tiles, r.top if gather else 0, N, K, _stream())


def activate(gu, act, limit, alpha, shift=1.0):
    """gu f32 [pairs, 2 F] (gate | up) -> act [pairs, F] = g sigmoid(alpha g) (u + shift) with g = min(gate,
    limit), u = clamp(up, -limit, limit). (limit inf, alpha 1, shift 0: silu(gate) up.)"""
    rows, two_f = gu.shape
    _check(gu, "gate_up", torch.float32, (rows, two_f))
    if two_f % 2:
        raise BackendError("moe activation: the input's width must be even")
    _check(act, "act", None, (rows, two_f // 2))
    lib.call("moe", "hb_moe_activate", gu.data_ptr(), act.data_ptr(), dtype_code(act), rows, two_f // 2, float(limit),
             float(alpha), float(shift), _stream())


def combine(y, routing, x, shared=None, gate=None, identity=None):
    """x[t] += sum_j weight[t, j] * y[row of pair (t, j)]; y f32 [pairs, H], x f32 [T, H].
    shared f32 [T, H] with gate = (f32 [T, ld], column): x[t] += sigmoid(gate[t, column]) * shared[t] as well.
    identity [T, H] (float32 or bfloat16): the experts' input rows, which are the output of a pair whose expert has
    no matrices (routing.real and beyond); needed where there are such experts."""
    r = routing
    H = x.shape[1]
    shared_ptr = gate_ptr = None
    gate_ld = 0
    if shared is not None:
        rows, column = gate
        _check(shared, "shared", torch.float32, (r.T, H))
        _check(rows, "gate", torch.float32, (r.T, None))
        gate_ld = rows.shape[1]
        if not 0 <= column < gate_ld:
            raise BackendError("moe combine: the gate's column lies outside its rows")
        shared_ptr, gate_ptr = shared.data_ptr(), rows.data_ptr() + 4 * column
    _check(y, "y", torch.float32, (r.T * r.top, H))
    _check(x, "x", torch.float32, (r.T, H))
    if r.real < r.E and identity is None:
        raise BackendError("moe combine: experts without matrices need the experts' input rows")
    if identity is not None:
        _check(identity, "identity", None, (r.T, H))
    lib.call("moe", "hb_moe_combine", y.data_ptr(), r.weight.data_ptr(), r.row_of.data_ptr(), x.data_ptr(), r.T,
             r.top, H, shared_ptr, gate_ptr, gate_ld, _ptr(identity) if r.real < r.E else None,
             0 if identity is None else dtype_code(identity), r.chosen.data_ptr(), r.real, _stream())


EPI_F32, EPI_BF16, EPI_GLU = 0, 1, 2
FEW_ROWS = 16      # up to so many rows a group the kernel without a stage in LDS runs (decoding)


def mfma_takes(K, lda, a_group_off=0, N=16):
    """True if the matrix-core kernel takes products of this inner size, layout and N weight rows
    (bfloat16 operands)."""
    return K % 32 == 0 and lda % 8 == 0 and a_group_off % 8 == 0 and N % 16 == 0


def pack_grouped(w):
    """[G, N, K] -> the same values with every W[g] in the matrix cores' operand order [K / 32, N / 16, 64, 8]
    (lane = 16 * (k / 8 % 4) + n % 16): what grouped_mfma reads."""
    G, N, K = w.shape
    if N % 16 or K % 32:
        raise BackendError("packed matrices need N in steps of 16 and K in steps of 32")
    return w.view(G, N // 16, 16, K // 32, 4, 8).permute(0, 3, 1, 4, 2, 5).contiguous().view(G, N, K)


def grouped_mfma(a, lda, a_group_off, w, c, ldc, c_group_off, epi, routing=None, gather=False, M=0, limit=0.0,
                 alpha=0.0, shift=1.0):
    """Group g: C[rows, g * c_group_off + n] = sum_k A[src(row), g * a_group_off + k] * w[g][n, k], bfloat16
    operands, float32 sums; w as pack_grouped gives it. With `routing` the rows are the (token, expert) pairs in their experts' order
    (gather: A's rows are the tokens'); without, every group takes the same M rows. epi: EPI_F32 / EPI_BF16
    store C in that type; EPI_GLU: w[g] is [2 F, K] (gate rows, then up rows) and C bfloat16 [*, F] receives
    the experts' activation with `limit`, `alpha` and `shift` (see activate)."""
    G, N, K = w.shape
    _check(a, "a", torch.bfloat16)
    _check(w, "w", torch.bfloat16, (G, N, K))
    _check(c, "c", torch.bfloat16 if epi != EPI_F32 else torch.float32)
    if not mfma_takes(K, lda, a_group_off, N) or (epi == EPI_GLU and N % 32):
        raise BackendError(f"grouped product: K = {K}, rows {lda} apart and groups {a_group_off} apart are not taken")
    out_cols = N // 2 if epi == EPI_GLU else N
    if routing is not None:
        r = routing
        rows_a, rows_c = (r.T if gather else r.T * r.top), r.T * r.top
        if G != r.real:
            raise BackendError("grouped product: one matrix an expert")
        lists = (r.order.data_ptr(), r.top if gather else 0, r.tile_expert.data_ptr(), r.tile_row0.data_ptr(),
                 r.tile_rows.data_ptr(), r.tiles, 0, 0)
        few = r.T * r.top <= FEW_ROWS * G          # (on average; the kernels take any tile either way)
    else:
        rows_a = rows_c = M
        lists = (None, 0, None, None, None, 0, M, G)
        few = M <= FEW_ROWS
    if (rows_a - 1) * lda + (G - 1) * a_group_off + K > a.numel() or \
            (rows_c - 1) * ldc + (G - 1) * c_group_off + out_cols > c.numel():
        raise BackendError("grouped product: an operand does not hold every row that is addressed")
    lib.call("moe", "hb_grouped_mfma", a.data_ptr(), lda, a_group_off, w.data_ptr(), N, K, c.data_ptr(), ldc,
             c_group_off, epi, *lists, float(limit), float(alpha), float(shift), 1 if few else 0, _stream())
