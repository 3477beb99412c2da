"""Each mechanism of the Bozasun decoder alone on the GPU against its plain formula: the attention's preparation
(biases, a norm a head with shared weights, rotation of pairs at divided rates, the cache's rows), the attention
over chunks of positions with capped scores (prompts in tiles of both heights, portions, single tokens across the
pages' and the chunks' edges, single keys made to stand out on either side of an edge and far back), the bias a
column, the state-space layer (filter with its bias, the walk whole, in portions down to one token and over
slots used again, memories long and short, the gated norm in groups), the experts' routing (softmax scores,
groups worth their best member, weights as they are, identity experts in the weighted sum) and the per-layer
token input."""
import math

import pytest
import torch

from herbert_rs_amd.cache import Cache, KVNeed, StateNeed
from herbert_rs_amd.kernels import mfma, moe, ops, recurrent
from herbert_rs_amd.parts.position import RotaryPairs

from .plain import bozasun as plain
from .test_vipalorn_kernels_gpu import step_meta

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def g(t):
    return None if t is None else t.to(DEV).contiguous()


def head_size(dtype, dim, vdim):
    size = max(dim, vdim)
    if dtype == torch.bfloat16:
        for takes in mfma.ATTENTION_HEAD_DIMS:
            if size <= takes:
                return takes
    return size


def attention_reference(proj, bias, qw, kw, rot, nq, nkv, dim, vdim, eps, scale, chunk, softcap, dtype):
    """(queries after bias, norm and rotation, the heads' outputs) by the plain formulas; bfloat16: queries, keys
    and values rounded as the cache holds them."""
    T = proj.shape[0]
    positions = torch.arange(T)
    p = proj + bias
    q = plain.rms_norm(p[:, :nq * dim].reshape(T, nq, dim), qw, eps)
    k = plain.rms_norm(p[:, nq * dim:(nq + nkv) * dim].reshape(T, nkv, dim), kw, eps)
    v = p[:, (nq + nkv) * dim:(nq + nkv) * dim + nkv * vdim].reshape(T, nkv, vdim)
    q, k = plain.rotate_pairs(q, positions, rot), plain.rotate_pairs(k, positions, rot)
    if dtype == torch.bfloat16:
        q, k, v = q.bfloat16().float(), k.bfloat16().float(), v.bfloat16().float()
    out = plain.masked_softmax_attention(q, k, v, plain.visible(positions, chunk), scale, softcap)
    return q, out.reshape(T, nq * vdim)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,dim,vdim,rot,chunk,softcap", [
    (6, 2, 24, 40, {"dims": 16, "base": 500.0, "scaling": {"factor": 5.0}}, 50, 8.0),
    (4, 4, 64, 64, {"dims": 64, "base": 10000.0}, 128, None),
    (8, 2, 64, 64, {"dims": 64, "base": 250000.0, "scaling": {"factor": 4.0}}, 100, 25.0),
    (2, 1, 160, 144, {"dims": 6, "base": 20.0, "scaling": {"factor": 3.0}}, 7, 50.0),
    (4, 2, 128, 128, None, 64, 15.0),
    (3, 3, 32, 32, {"dims": 32, "base": 100.0}, None, 4.0),
    (40, 1, 32, 32, {"dims": 8, "base": 100.0}, 33, 6.0),
])
def test_prepared_attention_over_chunks_with_capped_scores(nq, nkv, dim, vdim, rot, chunk, softcap, dtype):
    """A sequence of 230 tokens beside a short one, in portions and single tokens, three passes over slots that
    were used before, the prompt kernels' tiles of 64 and of 32 tokens asked for by name. In every head one channel
    is marked: the keys at a chunk's first position, at the position before it and far back are large there, and
    so are the queries behind them, so those keys hold the weight wherever they are seen: a chunk that starts
    one position early or late, or a far key that is missed, moves the output. That they do is checked on the
    plain formulas."""
    L, short, eps = 230, 9, 3e-6
    C = (nq + nkv) * dim + nkv * vdim
    proj = rand(L, C + 3, seed=1)
    bias = 0.5 * rand(C + 3, seed=6)
    bias[C:] = 0.0
    scale = 2.0 * dim ** -0.5
    edge = chunk if chunk else 70
    marked_k = [nq * dim + h * dim + dim - 1 for h in range(nkv)]
    marked_q = [h * dim + dim - 1 for h in range(nq)]
    for at in (5, edge - 1, edge, 2 * edge - 1, 2 * edge):
        if at < L:
            proj[at, marked_k] = 12.0
    proj[:, marked_q] = proj[:, marked_q].abs() + 3.0
    qw, kw = 1 + 0.2 * rand(dim, seed=3), 1 + 0.2 * rand(dim, seed=4)
    rot_dims = rot["dims"] if rot else 0
    q_ref, out_ref = attention_reference(proj[:, :C], bias[:C], qw, kw, rot, nq, nkv, dim, vdim, eps, scale, chunk, softcap, dtype)
    _, out_short = attention_reference(0.5 * proj[:short, :C], bias[:C], qw, kw, rot, nq, nkv, dim, vdim, eps, scale, chunk,
                                       softcap, dtype)
    # the marked keys do hold weight: with chunks one position longer, or without the cap, the output is another
    if chunk:
        _, other = attention_reference(proj[:, :C], bias[:C], qw, kw, rot, nq, nkv, dim, vdim, eps, scale, chunk + 1, softcap, dtype)
        assert float((other - out_ref).abs().max()) > 0.1 * float(out_ref.abs().max())
    if softcap and softcap <= 30.0:
        _, other = attention_reference(proj[:, :C], bias[:C], qw, kw, rot, nq, nkv, dim, vdim, eps, scale, chunk, None, dtype)
        assert float((other - out_ref).abs().max()) > 0.02 * float(out_ref.abs().max())
    hd = head_size(dtype, dim, vdim)
    cache = Cache({0: (KVNeed(nkv, hd, None),)}, 64 * 8, 4096, dtype, DEV, max_slots=3)
    kv = cache.kv_view(0)
    rates = None
    if rot is not None:
        sc = rot.get("scaling")
        part = RotaryPairs(rot["base"], rot_dims, None if sc is None else ("linear", sc["factor"]))
        rates = torch.tensor(part.pair_rates_host(), dtype=torch.float64, device=DEV)
    on_cores = dtype == torch.bfloat16
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
            ops.filter_norm_rotate_write(p, None, None, g(qw), g(kw), rates, rot_dims, meta, kv, q, nq, nkv, dim, vdim, hd, eps,
                                         bias=g(bias[:C]), head_norm=True)
            attn = torch.full_like(q, 9.0)
            if on_cores and mfma.attention_supported(q, kv, nq, nkv, hd):
                mfma.attention(q, meta, kv, attn, nq, nkv, hd, scale, 0, tile_height=height if meta.max_new > 1 else None,
                               chunk=chunk, softcap=softcap)
            else:
                ops.attention_plain(q, meta, kv, attn, nq, nkv, hd, scale, 0, chunk=chunk, softcap=softcap)
            out = attn.float().cpu().view(T, nq, hd)[..., :vdim].reshape(T, nq * vdim)
            got.append(out[:n_long])
            got_q.append(q[:n_long].float().cpu().view(n_long, nq, hd)[..., :dim])
            if n_short:
                got_short.append(out[n_long:])
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


def test_bias_a_column():
    x, b = rand(5, 77, seed=1), rand(77, seed=2)
    xg = x.to(DEV).clone()
    ops.add_bias(xg, b.to(DEV))
    assert torch.equal(xg.cpu(), x + b)


# ---------------------------------------------------------------- the state-space layer
@pytest.mark.parametrize("heads,P,N,groups,K,parts", [(1, 5, 8, 1, 1, 1), (3, 24, 10, 1, 3, 3), (4, 32, 16, 2, 4, 4), (6, 16, 64, 3, 2, 2),
                                                      (2, 64, 128, 2, 4, 1), (1, 80, 40, 1, 2, 2), (2, 20, 200, 1, 3, 1), (2, 12, 24, 1, 2, 1),
                                                      (8, 80, 16, 2, 3, 1)])
def test_state_space_layer_whole_in_portions_and_token_by_token(heads, P, N, groups, K, parts):
    """The rows [z | x | B | C | dt] as the projection leaves them: the filter with its bias and silu, the walk with
    decays near one (a long memory) and far below, the gate before the norm in groups."""
    inner, C = heads * P, heads * P + 2 * groups * N
    ld = 2 * inner + 2 * groups * N + heads
    lengths = [41, 3, 18]
    taps, conv_b = 1.0 / K + 0.3 * rand(C, K, seed=5), 0.3 * rand(C, seed=6)
    a_log = torch.tensor([-6.0, 0.5, -1.0, 0.2, -3.0, 0.0, -4.0, 0.3])[:heads]
    dt_bias, d_skip, norm_w = 0.3 * rand(heads, seed=7), 1 + 0.3 * rand(heads, seed=8), 1 + 0.2 * rand(inner, seed=9)
    projs = [rand(n, ld, seed=10 + i, scale=1.5) for i, n in enumerate(lengths)]

    def reference(p):
        T = p.shape[0]
        u = plain.silu(plain.causal_taps(p[:, inner:inner + C], taps, conv_b))
        x, B, Cm = (u[:, :inner].reshape(T, heads, P), u[:, inner:inner + groups * N].reshape(T, groups, N),
                    u[:, inner + groups * N:].reshape(T, groups, N))
        dt = plain.softplus(p[:, inner + C:] + dt_bias)
        y = plain.state_space_walk(x, B, Cm, dt, a_log, d_skip).reshape(T, inner)
        v = y * plain.silu(p[:, :inner])
        return u, y, (plain.rms_norm(v.view(T, parts, inner // parts), None, 1e-5).reshape(T, inner) * norm_w)

    refs = [reference(p) for p in projs]
    # the memory is long where the decay is near one: the first token still shows in the last output
    cut = projs[0].clone()
    cut[0] = 0.0
    assert float((reference(cut)[1][-1] - refs[0][1][-1]).abs().max()) > 1e-3
    needs = {0: (StateNeed((heads, recurrent.ssm_state_floats(N, P))), StateNeed((max(K - 1, 1), C)))}
    cache = Cache(needs, 64 * 8, 4096, torch.float32, DEV, max_slots=4)
    state, conv_state = cache.state_views(0)
    section = 256
    for cuts in ([], [1, 2, 3, 9, 17, 40], list(range(1, 41))):
        slots = [cache.alloc_slot() for _ in lengths]           # (slots that the round before has used: cleared)
        got = [[[], [], []] for _ in lengths]
        edges = sorted(set([0] + cuts + [max(lengths)]))
        for a, b in zip(edges[:-1], edges[1:]):
            live = [i for i, n in enumerate(lengths) if a < n]
            counts = [min(b, lengths[i]) - a for i in live]
            meta = step_meta(cache, [slots[i] for i in live], counts)
            proj = torch.cat([projs[i][a:a + c] for i, c in zip(live, counts)]).to(DEV).contiguous()
            T = proj.shape[0]
            u = torch.empty(T, C, device=DEV)
            recurrent.conv_silu(proj, g(taps), conv_state, meta, u, 0, 1, 0, 1.0, 0.0, -(-C // section), section, col0=inner,
                                bias=g(conv_b))
            y = torch.empty(T, inner, device=DEV)
            recurrent.ssm_scan(u, proj, inner + C, g(dt_bias), g(a_log), g(d_skip), state, meta, y, heads, groups, N, P)
            out = torch.empty(T, inner, device=DEV)
            recurrent.gated_group_norm(y, proj, 0, g(norm_w), out, parts, 1e-5)
            at = 0
            for i, c in zip(live, counts):
                for j, t in enumerate((u, y, out)):
                    got[i][j].append(t[at:at + c].cpu())
                at += c
        for i in range(len(lengths)):
            for j, (name, tol) in enumerate((("filter", 3e-6), ("walk", 2e-5), ("norm", 2e-5))):
                have, want = torch.cat(got[i][j]), refs[i][j]
                assert float((have - want).abs().max()) <= tol * max(1.0, float(want.abs().max())), f"{name}, cuts {cuts[:4]}"
        for s in slots:
            cache.free_slot(s)
    out = torch.empty(3, inner, dtype=torch.bfloat16, device=DEV)       # the norm's bfloat16 output
    p3 = projs[1].to(DEV)
    recurrent.gated_group_norm(g(refs[1][1]), p3, 0, g(norm_w), out, parts, 1e-5)
    assert torch.allclose(out.float().cpu(), refs[1][2], atol=3e-2, rtol=2e-2)


# ---------------------------------------------------------------- routing
@pytest.mark.parametrize("E,identity,top,groups", [(5, 2, 2, None), (9, 3, 3, (4, 2)), (6, 2, 3, (4, 3)), (3, 0, 3, None), (4, 2, 2, (6, 3)),
                                                   (70, 10, 6, (8, 3))])
def test_routing_by_softmax_scores_with_identity_experts(E, identity, top, groups):
    T, H, F = 37, 48, 16
    R = E + identity
    logits = rand(T, R + 3, seed=1, scale=2.0)
    correction = 0.05 * rand(R, seed=2) - 0.2          # (selection values may be negative: a group outside the kept ones must not win with 0)
    count, keep = groups if groups else (1, 1)
    routing = moe.Routing(torch.empty(moe.Routing.ints_needed(T, R, top), dtype=torch.int32, device=DEV),
                          torch.empty(T, top, device=DEV), T, R, top, real=E)
    moe.route(g(logits), g(correction), routing, scores=True, groups=count, keep=keep, score="softmax", worth_top=1, renorm=False)
    scores = torch.softmax(logits[:, :R], -1)
    chosen, weight = routing.chosen.view(T, top).cpu(), routing.weight.cpu()
    for t in range(T):
        want = plain.choose_experts(scores[t], correction, top, groups)
        assert chosen[t].tolist() == want, f"token {t}"
        assert torch.allclose(weight[t], scores[t][want], atol=1e-6)
    # the weighted sum: experts with matrices by the plain products over the tile list, identity experts the input itself
    y = rand(T, H, seed=3)
    gate_up = rand(E, 2 * F, H, seed=4, scale=H ** -0.5)
    down = rand(E, H, F, seed=5, scale=F ** -0.5)
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 3e-2)):
        yd = y.to(dtype)
        gu = torch.empty(T * top, 2 * F, device=DEV)
        moe.gemm_plain(g(yd), g(gate_up.to(dtype)), gu, routing, gather=True)
        act = torch.empty(T * top, F, dtype=dtype, device=DEV)
        moe.activate(gu, act, math.inf, 1.0, 0.0)
        out = torch.zeros(T * top, H, device=DEV)
        moe.gemm_plain(act, g(down.to(dtype)), out, routing, gather=False)
        x = torch.zeros(T, H, device=DEV)
        moe.combine(out, routing, x, identity=g(yd))
        want = torch.zeros(T, H)
        yf, wg, wd = yd.float(), gate_up.to(dtype).float(), down.to(dtype).float()
        for t in range(T):
            for j, e in enumerate(chosen[t].tolist()):
                if e < E:
                    a = plain.silu(yf[t] @ wg[e, :F].T) * (yf[t] @ wg[e, F:].T)
                    want[t] += weight[t, j] * (a.to(dtype).float() @ wd[e].T)
                else:
                    want[t] += weight[t, j] * yf[t]
        assert torch.allclose(x.cpu(), want, atol=tol, rtol=tol)


# ---------------------------------------------------------------- the per-layer token input
@pytest.mark.parametrize("T,H,D,layers,layer", [(1, 72, 5, 4, 3), (7, 176, 12, 6, 0), (3, 64, 1, 2, 1), (130, 512, 64, 3, 2), (2, 2052, 48, 2, 1)])
def test_token_input(T, H, D, layers, layer):
    V = 50
    x = rand(T, H, seed=1, scale=2.0)
    table, gate, proj = rand(V, layers * D, seed=2), rand(D, H, seed=3, scale=H ** -0.5), rand(H, D, seed=4)
    norm_w = 1 + 0.2 * rand(H, seed=5)
    tokens = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(6))
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 2e-5)):
        tb, gt, pj = table.to(dtype), gate.to(dtype), proj.to(dtype)
        want = plain.token_side(x, tb.float()[tokens][:, layer * D:(layer + 1) * D], {"gate": gt.float(), "proj": pj.float(), "norm": norm_w}, 1e-5)
        xg = x.to(DEV).clone()
        ops.token_side(xg, tokens.to(torch.int32).to(DEV), g(tb), layer * D, g(gt), g(pj.t()), g(norm_w), 1e-5,
                       torch.empty(T, D, device=DEV), torch.empty(T, H, device=DEV))
        assert float((xg.cpu() - want).abs().max()) <= tol * float(want.abs().max())
