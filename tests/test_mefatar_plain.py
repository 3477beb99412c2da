"""The plain Mefatar formulas pinned by library routines, by special cases that can be worked out by hand and by
invariants; the configuration, the parts' description and the cache's needs of the family, on the CPU."""
import json
import math

import pytest
import torch

from herbert_rs_amd.cache import KVNeed, StateNeed
from herbert_rs_amd.config.registry import resolve_architecture
from herbert_rs_amd.engine.model import Model
from herbert_rs_amd.errors import ConfigError
from herbert_rs_amd.parts.position import RotaryPairs

from .mefatar_tiny import CONFIGS
from .plain import mefatar as plain

F64 = torch.float64


def rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


def test_norm_and_activations_against_the_library():
    x, w = rand(5, 33), 1 + 0.1 * rand(33, seed=1)
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), torch.nn.functional.rms_norm(x, (33,), w, 1e-5), atol=1e-12)
    # eps lies inside the root
    assert math.isclose(float(plain.rms_norm(torch.tensor([3.0, 4.0], dtype=F64), torch.ones(2, dtype=F64), 2.0)[0]),
                        3.0 / math.sqrt(12.5 + 2.0))
    z = 3 * rand(200, seed=2)
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"), atol=1e-12)
    assert torch.allclose(plain.silu(z), torch.nn.functional.silu(z), atol=1e-12)
    assert torch.allclose(plain.softplus(10 * z), torch.nn.functional.softplus(10 * z), atol=1e-9)


def test_filter_against_the_library_and_by_hand():
    x, taps, bias = rand(9, 4), rand(4, 3, seed=2), rand(4, seed=3)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (2, 0)), taps[:, None, :], bias, groups=4)[0].T
    assert torch.allclose(plain.causal_filter(x, taps, bias), want, atol=1e-12)
    one = plain.causal_filter(torch.tensor([[1.0], [0.0], [0.0], [0.0]], dtype=F64), torch.tensor([[5.0, 7.0, 11.0]], dtype=F64))
    assert one[:, 0].tolist() == [11.0, 7.0, 5.0, 0.0]          # the last tap weighs the current token
    assert torch.equal(plain.causal_filter(x, torch.ones(4, 1, dtype=F64)), x)      # one tap: no filter


def test_rotation_rates_and_their_three_bands():
    r = {"dims": 8, "base": 100.0}
    plainly = plain.rotation_rates(r)
    assert torch.allclose(plainly, torch.tensor([100.0 ** (-2 * i / 8) for i in range(4)], dtype=F64))
    # wavelengths 2 pi / rate: 6.28, 19.9, 62.8, 198.7; original 64 with low 1 and high 4: under 16 stays, beyond
    # 64 is divided, between them the blend
    scaled = plain.rotation_rates(dict(r, scaling={"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}))
    assert scaled[0] == plainly[0] and math.isclose(float(scaled[3]), float(plainly[3]) / 8.0)
    for i in (1, 2):
        s = (64 / (2 * math.pi / float(plainly[i])) - 1.0) / (4.0 - 1.0)
        assert 0 < s < 1 and math.isclose(float(scaled[i]), (1 - s) * float(plainly[i]) / 8.0 + s * float(plainly[i]))
    # the engine's part gives the same rates
    part = RotaryPairs(100.0, 8, (8.0, 1.0, 4.0, 64))
    assert torch.allclose(torch.tensor(part.pair_rates_host(), dtype=F64), scaled, rtol=1e-14)
    assert torch.allclose(torch.tensor(RotaryPairs(100.0, 8).pair_rates_host(), dtype=F64), plainly, rtol=1e-14)


def test_rotation_turns_neighbouring_pairs_and_keeps_lengths():
    x = rand(7, 3, 10, seed=1)
    rates = plain.rotation_rates({"dims": 6, "base": 50.0})
    pos = torch.tensor([0, 1, 2, 5, 9, 100, 101])
    y = plain.rotate_pairs(x, pos, rates, 6)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 6:], x[..., 6:])         # position 0, and the entries past dims
    for i in range(3):
        assert torch.allclose((y[..., 2 * i:2 * i + 2] ** 2).sum(-1), (x[..., 2 * i:2 * i + 2] ** 2).sum(-1), atol=1e-12)
    a = float(pos[3]) * float(rates[1])                                            # by hand: pair 1 of position 5
    u, v = x[3, 0, 2], x[3, 0, 3]
    assert math.isclose(float(y[3, 0, 2]), float(u * math.cos(a) - v * math.sin(a)), abs_tol=1e-12)
    assert math.isclose(float(y[3, 0, 3]), float(v * math.cos(a) + u * math.sin(a)), abs_tol=1e-12)
    # scores depend on the difference of positions only
    q, k = rand(1, 1, 6, seed=2), rand(1, 1, 6, seed=3)
    dots = [float((plain.rotate_pairs(q, torch.tensor([p + 4]), rates, 6) * plain.rotate_pairs(k, torch.tensor([p]), rates, 6)).sum())
            for p in (0, 3, 77)]
    assert math.isclose(dots[0], dots[1], abs_tol=1e-10) and math.isclose(dots[0], dots[2], abs_tol=1e-10)


def test_attention_with_a_sink_against_the_library():
    """A sink is a key whose score is the sink itself (unscaled) and whose value is zero."""
    T, D, V = 9, 6, 5
    q, k, v = rand(T, D), rand(T, D, seed=1), rand(T, V, seed=2)
    for sink in (-1.5, 0.0, 2.5):
        got = plain.sink_attention(q, k, v, 0.37, torch.tensor(sink, dtype=F64))
        for i in range(T):
            s = torch.cat([(k[:i + 1] @ q[i]) * 0.37, torch.tensor([sink], dtype=F64)])
            p = torch.softmax(s, 0)
            assert torch.allclose(got[i], p[:-1] @ v[:i + 1], atol=1e-12)
    # a sink far below every score: the ordinary causal softmax attention
    lib = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True, scale=0.37)[0]
    assert torch.allclose(plain.sink_attention(q, k, v, 0.37, torch.tensor(-80.0, dtype=F64)), lib, atol=1e-12)
    # a sink far above: nothing is left for the values; the first row's weight is 1 / (1 + exp(sink - score))
    assert float(plain.sink_attention(q, k, v, 0.37, torch.tensor(60.0, dtype=F64)).abs().max()) < 1e-12
    first = plain.sink_attention(q, k, v, 1.0, torch.tensor(0.3, dtype=F64))[0]
    assert torch.allclose(first, v[0] / (1 + math.exp(0.3 - float(k[0] @ q[0]))), atol=1e-12)


def left_weights(W, m, seed=10):
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    w = {"q": rand(H * D, W, seed=seed), "k": rand(G * D, W, seed=seed + 1), "v": rand(G * V, W, seed=seed + 2),
         "g": rand(H * V, W, seed=seed + 3), "o": rand(W, H * V, seed=seed + 4), "sink": rand(H, seed=seed + 5),
         "q.norm": 1 + 0.1 * rand(H * D, seed=seed + 6), "k.norm": 1 + 0.1 * rand(G * D, seed=seed + 7)}
    if m.get("conv"):
        for name, rows in (("q", H * D), ("k", G * D), ("v", G * V)):
            w[name + ".conv"] = rand(rows, m["conv"], seed=seed + 8 + len(name) + rows)
    return w


def test_left_mixer_step_by_step_and_its_causality():
    T, W = 11, 16
    m = {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 10, "scale": 0.37, "conv": 3,
         "rot": {"dims": 4, "base": 30.0, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 16}}}
    w, h = left_weights(W, m), rand(T, W, seed=5)
    got = plain.left_mixer(h, w, m, 1e-5)
    # the same from library routines: filter, one norm over all heads, rotation, a zero-valued key for the sink
    def filt(x, taps):
        return torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (taps.shape[1] - 1, 0)), taps[:, None, :],
                                          groups=x.shape[1])[0].T
    q = torch.nn.functional.rms_norm(filt(h @ w["q"].T, w["q.conv"]), (24,), w["q.norm"], 1e-5).view(T, 4, 6)
    k = torch.nn.functional.rms_norm(filt(h @ w["k"].T, w["k.conv"]), (12,), w["k.norm"], 1e-5).view(T, 2, 6)
    v = filt(h @ w["v"].T, w["v.conv"]).view(T, 2, 10)
    rates = plain.rotation_rates(m["rot"])
    q, k = plain.rotate_pairs(q, torch.arange(T), rates, 4), plain.rotate_pairs(k, torch.arange(T), rates, 4)
    heads = []
    for n in range(4):
        s = (q[:, n] @ k[:, n // 2].T) * 0.37
        s = s.masked_fill(torch.arange(T)[None, :] > torch.arange(T)[:, None], -math.inf)
        p = torch.softmax(torch.cat([s, w["sink"][n].expand(T, 1)], 1), -1)[:, :-1]
        heads.append(p @ v[:, n // 2])
    o = torch.stack(heads, 1).reshape(T, 40) * torch.sigmoid(h @ w["g"].T)
    assert torch.allclose(got, o @ w["o"].T, atol=1e-9)
    h2 = h.clone()
    h2[7] += 1.0                                                   # a later token changes nothing before it
    assert torch.allclose(plain.left_mixer(h2, w, m, 1e-5)[:7], got[:7], atol=1e-12)
    # the norm runs over all heads at once: scaling one head's rows of W_q changes the other heads' queries
    w2 = dict(w, q=w["q"].clone())
    w2["q"][:6] *= 5.0
    assert not torch.allclose(plain.left_mixer(h, w2, m, 1e-5), got, atol=1e-3)


def test_decaying_state_special_cases():
    T, D, V = 6, 4, 3
    q, k, v = rand(T, D), rand(T, D, seed=1), rand(T, V, seed=2)
    keep, forget = torch.ones(T, D, dtype=F64), torch.zeros(T, D, dtype=F64)
    # no decay: causal linear attention, o_t = sum_{s <= t} (q_t . k_s) v_s
    want = torch.tril(q @ k.T) @ v
    assert torch.allclose(plain.decaying_state_attention(q, k, v, keep), want, atol=1e-12)
    # decay 0 in every channel forgets everything before the token (which the output still sees): o_t = (k_t . q_t) v_t
    assert torch.allclose(plain.decaying_state_attention(q, k, v, forget), (k * q).sum(-1)[:, None] * v, atol=1e-12)
    # the decay scales the rows of S that belong to key channels: channel 0 keeps, the others forget
    mixed = forget.clone()
    mixed[:, 0] = 1.0
    want = (torch.tril(q[:, :1] @ k[:, :1].T) @ v) + (k[:, 1:] * q[:, 1:]).sum(-1)[:, None] * v
    assert torch.allclose(plain.decaying_state_attention(q, k, v, mixed), want, atol=1e-12)
    # a constant decay a channel: the weight of token s at token t is prod_c alpha_c^(t - s) q_c k_c summed over channels
    alpha = torch.tensor([0.9, 0.5, 0.99, 0.2], dtype=F64).expand(T, D)
    want = torch.zeros(T, V, dtype=F64)
    for t in range(T):
        for s in range(t + 1):
            want[t] += (q[t] * k[s] * alpha[0] ** (t - s)).sum() * v[s]
    assert torch.allclose(plain.decaying_state_attention(q, k, v, alpha), want, atol=1e-12)


def test_right_mixer_its_decay_and_its_norm_a_head():
    T, W = 8, 12
    m = {"heads": 2, "dim": 4, "vdim": 6, "tau": 5.0}
    w = {"q": rand(8, W, seed=1), "k": rand(8, W, seed=2), "v": rand(12, W, seed=3), "g": rand(12, W, seed=4),
         "a1": rand(3, W, seed=5), "a2": rand(8, 3, seed=6), "a2.b": rand(8, seed=7), "norm": 1 + 0.1 * rand(6, seed=8),
         "o": rand(W, 12, seed=9)}
    h = rand(T, W, seed=10)
    got = plain.right_mixer(h, w, m, 1e-5)
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / 5.0).view(T, 2, 4)
    q, k, v = (h @ w["q"].T).view(T, 2, 4) * 0.5, (h @ w["k"].T).view(T, 2, 4), (h @ w["v"].T).view(T, 2, 6)
    o = torch.zeros(T, 2, 6, dtype=F64)
    for n in range(2):
        S = torch.zeros(4, 6, dtype=F64)
        for t in range(T):
            S = alpha[t, n][:, None] * S + k[t, n][:, None] * v[t, n][None, :]
            o[t, n] = q[t, n] @ S
    o = torch.nn.functional.rms_norm(o, (6,), w["norm"], 1e-5).reshape(T, 12) * torch.nn.functional.silu(h @ w["g"].T)
    assert torch.allclose(got, o @ w["o"].T, atol=1e-10)


def test_recurrent_unit_special_cases():
    T, C = 7, 5
    u = rand(T, C)
    lam = torch.tensor([-9.0, -2.0, 0.0, 1.0, 4.0], dtype=F64)
    ones, zeros = torch.ones(T, C, dtype=F64), torch.zeros(T, C, dtype=F64)
    # a closed gate on the decay (r = 0): a = 1, nothing enters, the state stays zero
    assert torch.equal(plain.gated_recurrence(u, zeros, ones, lam), zeros)
    # an open gate with a large softplus(lam) forgets at once: S_t = i_t u_t up to exp(-8 * 4)
    out = plain.gated_recurrence(u, ones, 0.5 * ones, torch.full((C,), 4.0, dtype=F64))
    assert torch.allclose(out, 0.5 * u, atol=1e-12)
    # the first token is no special case: S_0 = sqrt(1 - a^2) i u
    a = torch.exp(-8.0 * 0.3 * torch.nn.functional.softplus(lam))
    out = plain.gated_recurrence(u, 0.3 * ones, 0.7 * ones, lam)
    assert torch.allclose(out[0], torch.sqrt(1 - a * a) * 0.7 * u[0], atol=1e-12)
    assert torch.allclose(out[3], a * out[2] + torch.sqrt(1 - a * a) * 0.7 * u[3], atol=1e-12)
    # a constant input settles where the recurrence's fixed point lies
    long = plain.gated_recurrence(torch.ones(400, C, dtype=F64), 0.3 * torch.ones(400, C, dtype=F64),
                                  torch.ones(400, C, dtype=F64), lam)[-1]
    assert torch.allclose(long[1:], (torch.sqrt(1 - a * a) / (1 - a))[1:], rtol=1e-6)


def test_recurrent_mixer_step_by_step():
    T, W = 9, 10
    m = {"width": 6, "blocks": 3, "conv": 2}
    w = {"x": rand(6, W, seed=1), "x.b": rand(6, seed=2), "y": rand(6, W, seed=3), "y.b": rand(6, seed=4),
         "conv": rand(6, 2, seed=5), "conv.b": rand(6, seed=6), "ra": rand(3, 2, 2, seed=7), "ra.b": rand(3, 2, seed=8),
         "ri": rand(3, 2, 2, seed=9), "ri.b": rand(3, 2, seed=10), "lam": rand(6, seed=11), "o": rand(W, 6, seed=12)}
    h = rand(T, W, seed=13)
    got = plain.rglru_mixer(h, w, m)
    x = h @ w["x"].T + w["x.b"]
    u = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (1, 0)), w["conv"][:, None, :], w["conv.b"], groups=6)[0].T
    # the gates' matrices as one block-diagonal matrix
    r = torch.sigmoid(u @ torch.block_diag(*w["ra"]).T + w["ra.b"].reshape(-1))
    i = torch.sigmoid(u @ torch.block_diag(*w["ri"]).T + w["ri.b"].reshape(-1))
    S, rows = torch.zeros(6, dtype=F64), []
    for t in range(T):
        a = torch.exp(-8.0 * r[t] * torch.nn.functional.softplus(w["lam"]))
        S = a * S + torch.sqrt(1 - a * a) * i[t] * u[t]
        rows.append(S)
    y = torch.nn.functional.gelu(h @ w["y"].T + w["y.b"], approximate="tanh")
    assert torch.allclose(got, (torch.stack(rows) * y) @ w["o"].T, atol=1e-10)
    h2 = h.clone()
    h2[5] += 1.0
    assert torch.allclose(plain.rglru_mixer(h2, w, m)[:5], got[:5], atol=1e-12)


def test_the_order_in_which_layers_run():
    cfg = {"layers": [0] * 5}
    assert plain.layer_runs(cfg) == [0, 1, 2, 3, 4]
    assert plain.layer_runs(dict(cfg, loop={"start": 1, "stop": 3, "times": 3})) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert plain.layer_runs(dict(cfg, loop={"start": 0, "stop": 5, "times": 2})) == list(range(5)) * 2
    assert plain.layer_runs(dict(cfg, loop={"start": 2, "stop": 2, "times": 4})) == [0, 1, 2, 3, 4]
    assert plain.layer_runs(dict(cfg, loop={"start": 4, "stop": 5, "times": 1})) == [0, 1, 2, 3, 4]


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_configuration_spec_and_needs(name):
    raw = CONFIGS[name][0]
    arch = resolve_architecture(raw)
    cfg = arch.config_class.from_dict(raw)
    assert cfg.to_dict() == json.loads(json.dumps(raw))
    assert cfg.layer_runs() == plain.layer_runs(raw)
    spec = arch.build_spec(cfg)
    assert [e.layer for e in spec.schedule] == plain.layer_runs(raw)
    model = Model(spec)
    needs = model.tensor_needs()
    W = raw["width"]
    assert needs["embed"].shape == (raw["vocab"], W) and needs["final.norm"].shape == (W,)
    assert not any(k.startswith("lm_head") for k in needs)          # the head is the table itself
    cache_needs = model.cache_needs()
    runs = plain.layer_runs(raw)
    assert sorted(cache_needs) == list(range(len(runs)))             # a cache entry a run: every pass has its own
    for entry, i in enumerate(runs):
        layer, p = raw["layers"][i], f"l{i}."
        m = layer["mixer"]
        assert needs[p + "ls1"].shape == (W,) and needs[p + "norm1"].shape == (W,)
        assert (p + "norm2" in needs) == (p + "ls2" in needs) == (layer["mlp"] is not None)
        if layer["type"] == "rglru":
            n, b = m["width"], m["width"] // m["blocks"]
            assert needs[p + "mix.x"].shape == (n, W) and needs[p + "mix.y.b"].shape == (n,) and needs[p + "mix.o"].shape == (W, n)
            assert needs[p + "mix.ra"].shape == (m["blocks"], b, b) and needs[p + "mix.ri.b"].shape == (m["blocks"], b)
            assert needs[p + "mix.conv"].shape == (n, m["conv"]) and needs[p + "mix.lam"].shape == (n,)
            states = [StateNeed((n,), torch.float32)]
            if m["conv"] > 1:
                states.append(StateNeed((m["conv"] - 1, n), torch.float32))
            assert cache_needs[entry] == tuple(states)
        else:
            l, r = m["left"], m["right"]
            q, k, v = l["heads"] * l["dim"], l["kv_heads"] * l["dim"], l["kv_heads"] * l["vdim"]
            assert needs[p + "mix.left.q"].shape == (q, W) and needs[p + "mix.left.k.norm"].shape == (k,)
            assert needs[p + "mix.left.g"].shape == (l["heads"] * l["vdim"], W) and needs[p + "mix.left.sink"].shape == (l["heads"],)
            assert needs[p + "mix.left.out"].shape == (W,) and needs[p + "mix.right.out"].shape == (W,)
            assert (p + "mix.left.v.conv" in needs) == ("conv" in l)
            if "conv" in l:
                assert needs[p + "mix.left.v.conv"].shape == (v, l["conv"])
            assert needs[p + "mix.right.a2"].shape == (r["heads"] * r["dim"], r["rank"]) and needs[p + "mix.right.norm"].shape == (r["vdim"],)
            got = cache_needs[entry]
            assert got[0] == KVNeed(l["kv_heads"], max(l["dim"], l["vdim"]), None)
            want = []
            if l.get("conv", 1) > 1:
                want.append(StateNeed((l["conv"] - 1, q + k + v), torch.float32))
            want.append(StateNeed((r["heads"], r["dim"], r["vdim"]), torch.float32))
            assert list(got[1:]) == want
        if layer["mlp"] is not None:
            assert needs[p + "mlp.gate"].shape == (layer["mlp"]["ff"], W) and needs[p + "mlp.down"].shape == (W, layer["mlp"]["ff"])


def test_configuration_errors():
    base = CONFIGS["P"][0]
    arch = resolve_architecture(base)
    for path, value in ((("layers", 0, "type"), "conv"), (("layers", 0, "mlp", "kind"), "moe"), (("layers", 0, "mlp", "ff"), None),
                        (("layers", 0, "mixer", "left", "kv_heads"), 4), (("layers", 0, "mixer", "left", "scale"), None),
                        (("layers", 0, "mixer", "left", "rot", "dims"), 7), (("layers", 0, "mixer", "left", "rot", "dims"), 26),
                        (("layers", 0, "mixer", "left", "rot", "scaling", "high"), 1.0), (("layers", 0, "mixer", "right", "tau"), None),
                        (("layers", 0, "mixer", "right"), None), (("layers", 1, "mixer", "blocks"), 5), (("layers", 1, "mixer", "conv"), 0),
                        (("loop", "stop"), 4), (("loop", "times"), 0), (("loop", "start"), 4), (("norm",), None), (("vocab",), None),
                        (("width",), None)):
        raw = json.loads(json.dumps(base))
        at = raw
        for key in path[:-1]:
            at = at[key]
        if value is None:
            del at[path[-1]]
        else:
            at[path[-1]] = value
        with pytest.raises(ConfigError):
            arch.config_class.from_dict(raw)
            pytest.fail(f"{path} = {value} is taken")
    with pytest.raises(ConfigError):
        resolve_architecture({"architecture": "Mefatax"})


def test_sections_that_a_configuration_may_leave_out():
    """No "loop": every layer once; no "rank": the stored tensors give the middle's size; no "conv" and no "rot" on
    the attention: no filter, no rotation."""
    raw = json.loads(json.dumps(CONFIGS["S"][0]))
    del raw["loop"]
    del raw["layers"][1]["mixer"]["right"]["rank"]
    cfg = resolve_architecture(raw).config_class.from_dict(raw)
    assert cfg.loop is None and cfg.layer_runs() == [0, 1, 2]
    assert cfg.layers[1].mixer.right.rank is None and cfg.layers[2].mixer.left.rot is None
    assert resolve_architecture(CONFIGS["R"][0]).config_class.from_dict(CONFIGS["R"][0]).layers[0].mixer.left.conv is None
