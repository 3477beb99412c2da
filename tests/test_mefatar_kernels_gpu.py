"""Each mechanism of the Mefatar decoder alone on the GPU against its plain formula: the scaled sum before a
norm, the two normed outputs joined, the gated unit with the tanh form of gelu, the recurrent unit (its two
branches, the filter, the gates a block, the recurrence; whole, in portions down to one token, over slots that
are used again, memories long and short), the attention's preparation (filter, norm over the whole projection,
rotation of pairs with slowed wavelengths, the cache's rows) with the sink in the softmax and the gate after it
(prompts and single tokens across the pages' edges, one far key made to hold the weight, sinks large and
small), and the linear attention (the decay through its narrow middle, the state a head, the norm a head)."""
import math

import pytest
import torch

from herbert_rs_amd.cache import Cache, KVNeed, StateNeed
from herbert_rs_amd.kernels import mfma, ops, recurrent
from herbert_rs_amd.parts.position import RotaryPairs

from .plain import mefatar as plain
from .test_vipalorn_kernels_gpu import step_meta

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


# ---------------------------------------------------------------- sums, norms, the gated unit
@pytest.mark.parametrize("H", [24, 72, 1536, 2052, 4096])
def test_scaled_sum_then_norm(H):
    x, d, f, w = rand(7, H, seed=1, scale=2.0), rand(7, H, seed=2), 0.5 + 0.3 * rand(H, seed=3), 1 + 0.1 * rand(H, seed=4)
    want_x = x + f * d
    want_y = plain.rms_norm(want_x, w, 3e-6)
    for dtype, tol in ((torch.float32, 3e-6), (torch.bfloat16, 8e-3)):
        xg, y = x.to(DEV).clone(), torch.empty(7, H, dtype=dtype, device=DEV)
        ops.rmsnorm_scaled_sum(xg, d.to(DEV), f.to(DEV), w.to(DEV), y, 3e-6)
        assert torch.allclose(xg.cpu(), want_x, atol=1e-6, rtol=1e-6)
        assert torch.allclose(y.float().cpu(), want_y, atol=tol * 4, rtol=tol)
    xg = x.to(DEV).clone()                                              # the sum alone (a stack's last branch)
    ops.rmsnorm_scaled_sum(xg, d.to(DEV), f.to(DEV), None, None, 0.0)
    assert torch.allclose(xg.cpu(), want_x, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("H", [24, 72, 1536, 2052, 4096])
def test_two_normed_outputs_joined(H):
    a, b = rand(6, H, seed=1, scale=5.0), rand(6, H, seed=2, scale=0.2)            # of very different sizes
    wa, wb = 1 + 0.2 * rand(H, seed=3), 0.7 + 0.2 * rand(H, seed=4)
    want = 0.5 * plain.rms_norm(a, wa, 1e-5) + 0.25 * plain.rms_norm(b, wb, 1e-5)
    out = torch.full((6, H), 9.0, device=DEV)
    ops.normed_pair(a.to(DEV), wa.to(DEV), 0.5, b.to(DEV), wb.to(DEV), 0.25, out, 1e-5)
    assert torch.allclose(out.cpu(), want, atol=3e-6, rtol=3e-6)
    ops.normed_pair(a.to(DEV), wa.to(DEV), 0.5, b.to(DEV), wb.to(DEV), 0.25, out, 1e-5, accumulate=True)
    assert torch.allclose(out.cpu(), 2 * want, atol=6e-6, rtol=3e-6)


def test_gated_unit_with_the_tanh_form_of_gelu():
    gu = rand(5, 2 * 77, seed=3, scale=2.5)
    want = plain.gelu_tanh(gu[:, :77]) * gu[:, 77:]
    assert not torch.allclose(want, plain.silu(gu[:, :77]) * gu[:, 77:], atol=0.05)       # (the two forms differ visibly)
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 8e-3)):
        out = torch.empty(5, 77, dtype=dtype, device=DEV)
        ops.swiglu(gu.to(DEV), out, "gelu_tanh")
        assert torch.allclose(out.float().cpu(), want, atol=tol * 4, rtol=tol)


# ---------------------------------------------------------------- the recurrent unit
def unit_reference(proj, W, bx, by, taps, fb, r_w, r_b, i_w, i_b, lam):
    """In float64: where the decay is close to one, 1 - a^2 in float32 is only good to a few digits, and the
    kernel, which takes it from the decay's logarithm, is held to the exact value."""
    proj, bx, by, taps, fb, r_w, r_b, i_w, i_b, lam = (t.double() for t in (proj, bx, by, taps, fb, r_w, r_b, i_w, i_b, lam))
    u = plain.causal_filter(proj[:, :W] + bx, taps, fb)
    g = plain.gelu_tanh(proj[:, W:2 * W] + by)
    r = plain.sigmoid(plain.block_product(u, r_w, r_b))
    i = plain.sigmoid(plain.block_product(u, i_w, i_b))
    return u.float(), g.float(), (plain.gated_recurrence(u, r, i, lam) * g).float()


@pytest.mark.parametrize("W,blocks,K,lengths,all_cuts", [
    (8, 8, 1, [41, 3, 18], ([], [1, 2, 3, 9, 17, 40], list(range(1, 41)))),
    (96, 3, 4, [41, 3, 18], ([], [1, 2, 3, 9, 17, 40], list(range(1, 41)))),
    (40, 1, 2, [41, 3, 18], ([], [1, 2, 3, 9, 17, 40], list(range(1, 41)))),
    (256, 4, 3, [41, 3, 18], ([], [1, 2, 3, 9, 17, 40], list(range(1, 41)))),
    (192, 6, 4, [41, 3, 18], ([], [1, 2, 3, 9, 17, 40], list(range(1, 41)))),
    # portions of 128 tokens and more are walked as sixteen runs side by side: lengths that the runs divide and
    # do not, a sequence shorter than the number of runs beside a long one, a long portion after a short one
    (96, 3, 4, [333, 5, 140], ([], [130], [2, 131, 132, 260])),
    (72, 2, 2, [128, 128, 1], ([], [127])),
])
def test_recurrent_unit_whole_in_portions_and_token_by_token(W, blocks, K, lengths, all_cuts):
    """Portions shorter than the filter's taps, single tokens, sequences of unequal lengths in one step, slots
    that the pass before used; rates from memories of a few tokens to ones that outlast the sequence."""
    b = W // blocks
    ld = 2 * W + 5
    bx, by, fb = 0.3 * rand(W, seed=1), 0.3 * rand(W, seed=2), 0.2 * rand(W, seed=3)
    taps = 1.0 / K + 0.3 * rand(W, K, seed=4)
    r_w, i_w = rand(blocks, b, b, seed=5) / b ** 0.5, rand(blocks, b, b, seed=6) / b ** 0.5
    r_b, i_b = 0.3 * rand(blocks, b, seed=7), 0.3 * rand(blocks, b, seed=8)
    lam = torch.linspace(-8.0, 1.0, W)
    projs = [rand(n, ld, seed=10 + i, scale=1.5) for i, n in enumerate(lengths)]
    refs = [unit_reference(p, W, bx, by, taps, fb, r_w, r_b, i_w, i_b, lam) for p in projs]
    gate_w = torch.cat([r_w, i_w], 1).contiguous().to(DEV)                # [blocks, 2 b, b]
    cache = Cache({0: (StateNeed((W,)), StateNeed((max(K - 1, 1), W)))}, 64 * 16, 4096, torch.float32, DEV, max_slots=4)
    state, conv_state = cache.state_views(0)
    g = lambda t: t.reshape(-1).contiguous().to(DEV)
    for cuts in all_cuts:
        slots = [cache.alloc_slot() for _ in lengths]
        got = [[] for _ in lengths]
        edges = sorted(set([0] + cuts + [max(lengths)]))
        for a, e in zip(edges[:-1], edges[1:]):
            live = [i for i, n in enumerate(lengths) if a < n]
            counts = [min(e, lengths[i]) - a for i in live]
            meta = step_meta(cache, [slots[i] for i in live], counts)
            proj = torch.cat([projs[i][a:a + c] for i, c in zip(live, counts)]).to(DEV).contiguous()
            T = proj.shape[0]
            ug = torch.empty(T, 2 * W, device=DEV)
            recurrent.lru_inputs(proj, g(bx), g(by), taps.to(DEV), g(fb), conv_state, meta, ug)
            gates = torch.empty(T, 2 * W, device=DEV)
            ops.gemm_plain_batched(ug, gate_w, gates, T, 2 * b, b, 2 * W, b, 2 * W, blocks, b, 2 * b * b, 2 * b)
            out = torch.empty(T, W, device=DEV)
            recurrent.lru_scan(ug, gates, g(r_b), g(i_b), lam.to(DEV), 8.0, state, meta, out, b)
            at = 0
            for i, c in zip(live, counts):
                got[i].append((ug[at:at + c].cpu(), out[at:at + c].cpu()))
                at += c
        for i in range(len(lengths)):
            ug = torch.cat([p[0] for p in got[i]])
            assert torch.allclose(ug[:, :W], refs[i][0], atol=3e-6), f"filter, cuts {cuts[:4]}"
            assert torch.allclose(ug[:, W:], refs[i][1], atol=3e-6), f"gelu branch, cuts {cuts[:4]}"
            assert torch.allclose(torch.cat([p[1] for p in got[i]]), refs[i][2], atol=1e-5, rtol=1e-5), f"recurrence, cuts {cuts[:4]}"
        for s in slots:
            cache.free_slot(s)


def test_recurrent_unit_remembers_its_first_token():
    """A rate near zero: the first token's input, which enters through sqrt(1 - a^2) like any other (the state
    before it is zero), is still most of the state 300 tokens later, after 299 single-token steps."""
    W, L = 64, 300
    lam = torch.full((W,), -12.0)
    u = torch.zeros(L, W)
    u[0] = 100.0 * (1 + rand(W, seed=1).abs())
    gates = torch.zeros(L, 2 * W)
    ug = torch.cat([u, torch.ones(L, W)], 1)
    half = torch.full((L, W), 0.5, dtype=torch.float64)
    want = plain.gated_recurrence(u.double(), half, half, lam.double()).float()
    assert float(want[-1].abs().min()) > 0.9 * float(want[0].abs().min()) > 0
    cache = Cache({0: (StateNeed((W,)),)}, 64 * 8, 4096, torch.float32, DEV, max_slots=2)
    state = cache.state_views(0)[0]
    slot = cache.alloc_slot()
    zeros = torch.zeros(W, device=DEV)
    rows = []
    for t in range(L):
        meta = step_meta(cache, [slot], [1])
        out = torch.empty(1, W, device=DEV)
        recurrent.lru_scan(ug[t:t + 1].to(DEV).contiguous(), gates[t:t + 1].to(DEV).contiguous(), zeros, zeros, lam.to(DEV), 8.0,
                           state, meta, out, W)
        rows.append(out.cpu())
    assert torch.allclose(torch.cat(rows), want, rtol=2e-5, atol=1e-7)


# ---------------------------------------------------------------- the attention: preparation, sink, gate
def head_size(dtype, dim, vdim):
    size = max(dim, vdim)
    if dtype == torch.bfloat16:
        for takes in mfma.ATTENTION_HEAD_DIMS:
            if size <= takes:
                return takes
    return size


def attention_reference(proj, taps, qw, kw, rot, sinks, nq, nkv, dim, vdim, eps, scale, dtype):
    """Queries, keys and values as the kernels store them (rounded to `dtype`) and the gated heads [L, nq vdim]."""
    L = proj.shape[0]
    C = (nq + nkv) * dim + nkv * vdim
    x = proj[:, :C] if taps is None else plain.causal_filter(proj[:, :C], taps)
    q = plain.rms_norm(x[:, :nq * dim], qw, eps).view(L, nq, dim)
    k = plain.rms_norm(x[:, nq * dim:(nq + nkv) * dim], kw, eps).view(L, nkv, dim)
    v = x[:, (nq + nkv) * dim:].view(L, nkv, vdim)
    if rot is not None:
        rates = plain.rotation_rates(rot)
        q, k = plain.rotate_pairs(q, torch.arange(L), rates, rot["dims"]), plain.rotate_pairs(k, torch.arange(L), rates, rot["dims"])
    q, k, v = (t.to(dtype).float() for t in (q, k, v))
    heads = [plain.sink_attention(q[:, h], k[:, h // (nq // nkv)], v[:, h // (nq // nkv)], scale, sinks[h]) for h in range(nq)]
    o = torch.stack(heads, 1).to(dtype).float().reshape(L, nq * vdim)
    return q, o * plain.sigmoid(proj[:, C:C + nq * vdim])


CASES = [  # nq, nkv, dim, vdim, K, rotation, sinks' size
    (4, 2, 64, 64, 4, {"dims": 64, "base": 10000.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}, 1.0),
    (6, 2, 24, 40, 3, {"dims": 16, "base": 500.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}, 4.0),
    (1, 1, 48, 80, 0, {"dims": 48, "base": 50.0}, 0.5),
    (2, 1, 160, 144, 2, {"dims": 6, "base": 20.0, "scaling": {"factor": 2.0, "low": 0.5, "high": 3.0, "original": 32}}, 2.0),
    (8, 2, 128, 128, 4, None, 6.0),
    (3, 3, 32, 16, 1, {"dims": 8, "base": 100.0}, -3.0),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,dim,vdim,K,rot,sink_size", CASES)
def test_prepared_attention_with_a_sink_and_a_far_key(nq, nkv, dim, vdim, K, rot, sink_size, dtype):
    """A prompt of 150 tokens in portions (2, 61, 2, 85: a portion shorter than the taps, edges beside a page's),
    then single tokens to 215, beside a short sequence in the same steps. Where a head has entries that do not
    turn, the keys of positions 5 and 64 (a page's first place) and all queries from 100 on carry a large
    value there (scores three times as sharp), so that those two keys hold most of those queries' weight,
    whatever lies between."""
    eps, L, short = 2e-6, 215, 9
    C = (nq + nkv) * dim + nkv * vdim
    ld = C + nq * vdim + 3
    proj = rand(L, ld, seed=dim + K)
    rot_dims = 0 if rot is None else rot["dims"]
    far = rot_dims < dim
    scale = (3.0 if far else 1.3) * dim ** -0.5
    taps = None if K == 0 else 1.0 / K + 0.3 * rand(C, K, seed=2)
    if far:
        marked = [nq * dim + h * dim + dim - 1 for h in range(nkv)] + [h * dim + dim - 1 for h in range(nq)]
        proj[5, marked[:nkv]] = proj[64, marked[:nkv]] = 20.0
        proj[100:, marked[nkv:]] = 6.0
        if taps is not None:             # the marked channels pass the filter unchanged, so that the mark stays on its token
            taps[marked] = 0.0
            taps[marked, K - 1] = 1.0
    qw, kw = 1 + 0.2 * rand(nq * dim, seed=3), 1 + 0.2 * rand(nkv * dim, seed=4)
    sinks = sink_size * (0.5 + rand(nq, seed=5).abs())
    q_ref, out_ref = attention_reference(proj, taps, qw, kw, rot, sinks, nq, nkv, dim, vdim, eps, scale, dtype)
    _, out_short = attention_reference(0.5 * proj[:short], taps, qw, kw, rot, sinks, nq, nkv, dim, vdim, eps, scale, dtype)
    if far:                              # the far keys do hold the weight: without them the output is another
        gone = proj.clone()
        gone[[5, 64]] = 0.0
        _, other = attention_reference(gone, taps, qw, kw, rot, sinks, nq, nkv, dim, vdim, eps, scale, dtype)
        assert float((other[150:] - out_ref[150:]).abs().max()) > 0.1 * float(out_ref[150:].abs().max())
    hd = head_size(dtype, dim, vdim)
    needs = (KVNeed(nkv, hd, None),) + ((StateNeed((K - 1, C)),) if K > 1 else ())
    cache = Cache({0: needs}, 64 * 8, 4096, dtype, DEV, max_slots=3)
    kv = cache.kv_view(0)
    state = cache.state_views(0)[0] if K > 1 else None
    rates = None
    if rot is not None:
        sc = rot.get("scaling")
        part = RotaryPairs(rot["base"], rot_dims, None if sc is None else (sc["factor"], sc["low"], sc["high"], sc["original"]))
        rates = torch.tensor(part.pair_rates_host(), dtype=torch.float64, device=DEV)
    g = lambda t: None if t is None else t.to(DEV).contiguous()
    # three passes: the later ones find the slots, pages and filter rows used, and ask the matrix cores' prompt kernels
    # for their tiles of 64 and of 32 tokens by name (the first pass leaves the choice to the host)
    for again, height in enumerate((None, 64, 32)):
        a, b = cache.alloc_slot(), cache.alloc_slot()
        got, got_short, got_q = [], [], []
        steps = [(2, 2), (61, 3), (2, 1), (85, 3)] + [(1, 0)] * (L - 150)
        done = done_short = 0
        for n_long, n_short in steps:
            slots, counts = ([a, b], [n_long, n_short]) if n_short else ([a], [n_long])
            meta = step_meta(cache, slots, counts)
            p = torch.cat([proj[done:done + n_long]] + ([0.5 * proj[done_short:done_short + n_short]] if n_short else []))
            p = p.to(DEV).contiguous()
            T = p.shape[0]
            q = torch.empty(T, nq * hd, dtype=dtype, device=DEV)
            ops.filter_norm_rotate_write(p, g(taps), state, g(qw), g(kw), rates, rot_dims, meta, kv, q, nq, nkv, dim, vdim, hd, eps)
            attn = torch.full_like(q, 9.0)
            if dtype == torch.bfloat16 and mfma.attention_supported(q, kv, nq, nkv, hd):
                mfma.attention(q, meta, kv, attn, nq, nkv, hd, scale, 0, sinks=g(sinks), tile_height=height if meta.max_new > 1 else None)
            else:
                ops.attention_plain(q, meta, kv, attn, nq, nkv, hd, scale, 0, sinks=g(sinks))
            gated = torch.empty(T, nq * vdim, dtype=dtype, device=DEV)
            ops.gate_heads(attn, p, C, gated, nq, hd, vdim)
            got.append(gated[:n_long].float().cpu())
            got_q.append(q[:n_long].float().cpu().view(n_long, nq, hd)[..., :dim])
            if n_short:
                got_short.append(gated[n_long:].float().cpu())
            done, done_short = done + n_long, done_short + n_short
        got, got_short, got_q = torch.cat(got), torch.cat(got_short), torch.cat(got_q)
        tol = 2e-5 if dtype == torch.float32 else 2 ** -6
        err_q = (got_q - q_ref).abs().amax((-1, -2))
        assert float(err_q.max()) <= (1e-5 if dtype == torch.float32 else 2 ** -7) * float(q_ref.abs().max()), \
            f"queries, position {int(err_q.argmax())}"
        err = (got - out_ref).abs().max(-1).values
        assert float(err.max()) <= tol * float(out_ref.abs().max()), f"pass {again}: worst at position {int(err.argmax())}"
        assert float((got_short - out_short).abs().max()) <= tol * float(out_short.abs().max()), f"pass {again}: the short one"
        cache.free_slot(a)
        cache.free_slot(b)


# ---------------------------------------------------------------- the linear attention
@pytest.mark.parametrize("heads,D,V,rank,tau", [(1, 16, 80, 5, 1.0), (3, 24, 40, 10, 7.0), (2, 32, 32, 16, 16.0), (2, 22, 48, 12, 3.0),
                                                (4, 64, 128, 32, 16.0)])
def test_linear_attention_its_decay_and_its_norm_a_head(heads, D, V, rank, tau):
    """The rows [q | k | v | g | middle] as the projection leaves them; the decay's second product with its
    sigmoid and root, the state a head over portions and single tokens and slots used again, the norm a head
    with silu of the gate."""
    qk, hv = heads * D, heads * V
    g_off, a_off = 2 * qk + hv, 2 * qk + 2 * hv
    ld = a_off + rank
    lengths = [41, 3, 18]
    a2, a2_b = rand(qk, rank, seed=1, scale=1.5 / rank ** 0.5).bfloat16().float(), 2.0 + rand(qk, seed=2)
    norm_w = 1 + 0.2 * rand(V, seed=3)
    projs = [rand(n, ld, seed=20 + i) for i, n in enumerate(lengths)]

    def reference(p):
        T = p.shape[0]
        q, k = (p[:, :qk] * D ** -0.5).view(T, heads, D), p[:, qk:2 * qk].view(T, heads, D)
        v = p[:, 2 * qk:2 * qk + hv].view(T, heads, V)
        alpha = (plain.sigmoid(p[:, a_off:] @ a2.T + a2_b) ** (1.0 / tau)).view(T, heads, D)
        o = torch.stack([plain.decaying_state_attention(q[:, h], k[:, h], v[:, h], alpha[:, h]) for h in range(heads)], 1)
        return alpha.reshape(T, qk), (plain.rms_norm(o, norm_w, 1e-5).reshape(T, hv) * plain.silu(p[:, g_off:g_off + hv]))
    refs = [reference(p) for p in projs]
    cache = Cache({0: (StateNeed((heads, D, V)),)}, 64 * 8, 4096, torch.float32, DEV, max_slots=4)
    state = cache.state_views(0)[0]
    for cuts in ([], [1, 2, 3, 9, 17, 40], list(range(1, 41))):
        slots = [cache.alloc_slot() for _ in lengths]
        got = [[] for _ in lengths]
        edges = sorted(set([0] + cuts + [max(lengths)]))
        for a, e in zip(edges[:-1], edges[1:]):
            live = [i for i, n in enumerate(lengths) if a < n]
            counts = [min(e, lengths[i]) - a for i in live]
            meta = step_meta(cache, [slots[i] for i in live], counts)
            proj = torch.cat([projs[i][a:a + c] for i, c in zip(live, counts)]).to(DEV).contiguous()
            T = proj.shape[0]
            decay = torch.empty(T, qk, device=DEV)
            ops.gemm_plain_columns(proj, a_off, rank, a2.to(DEV), decay, decay=("sigmoid_root", a2_b.to(DEV), 1.0 / tau))
            o = torch.empty(T, hv, device=DEV)
            recurrent.gated_delta(proj, None, 0, 0, None, None, state, meta, o, heads, heads, D, V, decay=decay, correction=False,
                                  out_scale=D ** -0.5)
            out = torch.empty(T, hv, device=DEV)
            recurrent.gated_head_norm(o, proj, g_off, norm_w.to(DEV), out, heads, V, 1e-5, gate="silu")
            at = 0
            for i, c in zip(live, counts):
                got[i].append((decay[at:at + c].cpu(), out[at:at + c].cpu()))
                at += c
        for i in range(len(lengths)):
            assert torch.allclose(torch.cat([p[0] for p in got[i]]), refs[i][0], atol=3e-6), f"decay, cuts {cuts[:4]}"
            assert torch.allclose(torch.cat([p[1] for p in got[i]]), refs[i][1], atol=2e-5, rtol=2e-5), f"state and norm, cuts {cuts[:4]}"
        for s in slots:
            cache.free_slot(s)


def test_linear_attention_keeps_a_far_token():
    """Decays of one on one channel and of a half on the others: 200 single-token steps later the first token's
    value is what a query on that channel reads, and nothing of it is left on the others."""
    D, V, L = 8, 16, 200
    q, k, v = torch.zeros(L, D), torch.zeros(L, D), rand(L, V, seed=1)
    k[0, 3] = 1.0
    k[1:, 5] = 1.0
    q[:, 3] = 1.0
    alpha = torch.full((L, D), 0.5)
    alpha[:, 3] = 1.0
    want = plain.decaying_state_attention(q, k, v, alpha)
    assert torch.allclose(want[-1], v[0])
    cache = Cache({0: (StateNeed((1, D, V)),)}, 64 * 8, 4096, torch.float32, DEV, max_slots=2)
    state = cache.state_views(0)[0]
    slot = cache.alloc_slot()
    rows = torch.cat([q, k, v], 1)
    out = []
    for t in range(L):
        meta = step_meta(cache, [slot], [1])
        o = torch.empty(1, V, device=DEV)
        recurrent.gated_delta(rows[t:t + 1].to(DEV).contiguous(), None, 0, 0, None, None, state, meta, o, 1, 1, D, V,
                              decay=alpha[t:t + 1].to(DEV).contiguous(), correction=False)
        out.append(o.cpu())
    assert torch.allclose(torch.cat(out), want, atol=1e-6)
