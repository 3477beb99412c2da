"""The plain formulas of the Bozasun decoder checked against independent ones on the CPU, and the configuration:
what the engine is compared with on the GPU has to be right by itself."""
import json
import math

import pytest
import torch

import herbert_rs_amd as hb
from herbert_rs_amd.config import BozasunConfig
from herbert_rs_amd.config.registry import resolve_architecture
from herbert_rs_amd.engine.model import Model
from herbert_rs_amd.errors import ConfigError

from .bozasun_tiny import CONFIGS, make_folder, random_tokens
from .plain import bozasun as plain


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


def test_chunks_count_from_the_sequence_start():
    pos = torch.arange(23)
    see = plain.visible(pos, 5)
    for i in range(23):
        for j in range(23):
            assert bool(see[i, j]) == (j <= i and i // 5 == j // 5)
    assert bool(plain.visible(pos, None)[22, 0]) and not bool(plain.visible(pos, None)[0, 1])
    # a portion that starts in the middle of a chunk keeps the sequence's own chunks
    assert torch.equal(plain.visible(torch.arange(7, 14), 5), see[7:14, 7:14])


def test_pairs_turn_by_the_difference_of_positions():
    rot = {"dims": 6, "base": 50.0, "scaling": {"factor": 4.0}}
    q, k = rand(1, 1, 10, seed=1), rand(1, 1, 10, seed=2)
    a = (plain.rotate_pairs(q, torch.tensor([9]), rot) * plain.rotate_pairs(k, torch.tensor([4]), rot)).sum()
    b = (plain.rotate_pairs(q, torch.tensor([105]), rot) * plain.rotate_pairs(k, torch.tensor([100]), rot)).sum()
    assert abs(float(a - b)) < 1e-9
    turned = plain.rotate_pairs(q, torch.tensor([9]), rot)
    assert torch.equal(turned[..., 6:], q[..., 6:])                      # the rest passes unchanged
    assert abs(float(turned.norm() - q.norm())) < 1e-12
    # pair 0 of position 1 turns by 1 / factor; the scaling divides every rate
    unit = torch.zeros(1, 1, 10, dtype=torch.float64)
    unit[0, 0, 0] = 1.0
    t = plain.rotate_pairs(unit, torch.tensor([1]), rot)
    assert abs(float(t[0, 0, 0]) - math.cos(0.25)) < 1e-12 and abs(float(t[0, 0, 1]) - math.sin(0.25)) < 1e-12
    rates = plain.pair_rates({"dims": 6, "base": 50.0})
    assert torch.allclose(plain.pair_rates(rot) * 4.0, rates) and abs(float(rates[2]) - 50.0 ** (-4 / 6)) < 1e-12


def test_pairs_are_halves_of_reordered_entries():
    """What the latent attention's loader relies on: a dot product of two vectors whose neighbouring pairs were turned
    equals that of the same vectors with entries in the order (even, odd), turned as halves."""
    rot = {"dims": 8, "base": 100.0}
    q, k = rand(3, 1, 8, seed=3), rand(3, 1, 8, seed=4)
    pos = torch.tensor([2, 50, 7])
    want = (plain.rotate_pairs(q, pos, rot) * plain.rotate_pairs(k, pos.flip(0), rot)).sum(-1)
    order = torch.cat([torch.arange(0, 8, 2), torch.arange(1, 8, 2)])

    def halves(x, p):
        ang = p.double()[:, None] * plain.pair_rates(rot)[None, :]
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        a, b = x[..., :4], x[..., 4:]
        return torch.cat([a * c - b * s, b * c + a * s], -1)
    got = (halves(q[..., order], pos) * halves(k[..., order], pos.flip(0))).sum(-1)
    assert torch.allclose(got, want, atol=1e-12)


def test_capped_scores_and_the_softmax_within_a_chunk():
    T, D = 9, 4
    q, k, v = rand(T, 2, D, seed=1, scale=3.0), rand(T, 1, D, seed=2, scale=3.0), rand(T, 1, 3, seed=3)
    see = plain.visible(torch.arange(T), 4)
    out = plain.masked_softmax_attention(q, k, v, see, 0.7, 2.5)
    for h in range(2):
        for i in range(T):
            js = [j for j in range(T) if j <= i and j // 4 == i // 4]
            s = torch.tensor([2.5 * math.tanh(0.7 * float(q[i, h] @ k[j, 0]) / 2.5) for j in js], dtype=torch.float64)
            assert s.abs().max() <= 2.5
            w = torch.exp(s - s.max())
            want = sum(w[n] / w.sum() * v[j, 0] for n, j in enumerate(js))
            assert torch.allclose(out[i, h], want, atol=1e-12)
    assert torch.allclose(out[4], v[4, 0].expand(2, 3))                 # a chunk's first query sees its own key alone


def test_state_space_walk_is_the_sum_over_the_past():
    T, H, P, G, N = 7, 2, 3, 1, 4
    x, B, C = rand(T, H, P, seed=1), rand(T, G, N, seed=2), rand(T, G, N, seed=3)
    dt, a_log, d = rand(T, H, seed=4).abs() + 0.1, torch.tensor([-1.0, 0.3], dtype=torch.float64), rand(H, seed=5)
    y = plain.state_space_walk(x, B, C, dt, a_log, d)
    for h in range(H):
        for t in range(T):
            want = d[h] * x[t, h]
            for s in range(t + 1):
                decay = math.exp(-math.exp(float(a_log[h])) * float(dt[s + 1:t + 1, h].sum()))
                want = want + decay * float(dt[s, h]) * float(C[t, 0] @ B[s, 0]) * x[s, h]
            assert torch.allclose(y[t, h], want, atol=1e-12)


def test_filter_is_a_causal_convolution_with_a_bias():
    u, taps, bias = rand(11, 5, seed=1), rand(5, 3, seed=2), rand(5, seed=3)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(u.T[None], (2, 0)), taps[:, None, :], bias, groups=5)[0].T
    assert torch.allclose(plain.causal_taps(u, taps, bias), want, atol=1e-12)


def test_the_choice_of_experts():
    s = torch.tensor([0.30, 0.05, 0.20, 0.10, 0.25, 0.10], dtype=torch.float64)
    zero = torch.zeros(6, dtype=torch.float64)
    assert plain.choose_experts(s, zero, 2, None) == [0, 4]
    # groups of neighbours, worth their best member: (0.30, 0.20, 0.25); the two best are the first and the last
    assert plain.choose_experts(s, zero, 3, (3, 2)) == [0, 4, 5]
    # the correction moves the choice, not the score; selection values may be negative, and an expert outside the
    # kept groups is never chosen, whatever 0 would compare to
    c = torch.tensor([-1.0, -1.0, -0.85, -1.0, -2.0, -2.0], dtype=torch.float64)
    assert plain.choose_experts(s, c, 2, (3, 1)) == [2, 3]             # the groups are worth -0.70, -0.65 and -1.75
    assert plain.choose_experts(s, c, 2, (3, 2)) == [2, 0]             # both of the first two groups: -0.65, then -0.70
    assert plain.choose_experts(torch.tensor([0.5, 0.5], dtype=torch.float64), torch.zeros(2, dtype=torch.float64), 1, None) == [0]


def test_identity_experts_pass_their_input_on():
    H, F = 6, 4
    h = rand(3, H, seed=1)
    mlp = {"kind": "moe", "expert": {"ff": F}, "router": {"experts": 2, "identity": 2, "top": 4}}
    w = {"router": rand(4, H, seed=2), "correction": rand(4, seed=3)}
    for e in range(2):
        w.update({f"e{e}.gate": rand(F, H, seed=10 + e), f"e{e}.up": rand(F, H, seed=20 + e), f"e{e}.down": rand(H, F, seed=30 + e)})
    s = torch.softmax(h @ w["router"].T, -1)
    want = sum(s[:, e:e + 1] * plain.gated_unit(h, w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"]) for e in range(2))
    want = want + (s[:, 2:3] + s[:, 3:4]) * h                            # weights are the scores as they are: they add up to 1 here
    assert torch.allclose(plain.moe_ff(h, w, mlp), want, atol=1e-12)


def test_token_input_reads_the_stream_itself():
    x, rows = rand(4, 6, seed=1), rand(4, 2, seed=2)
    w = {"gate": rand(2, 6, seed=3), "proj": rand(6, 2, seed=4), "norm": rand(6, seed=5)}
    z = x @ w["gate"].T
    g = 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3))) * rows
    y = g @ w["proj"].T
    want = x + y / torch.sqrt((y * y).mean(-1, keepdim=True) + 1e-5) * w["norm"]
    assert torch.allclose(plain.token_side(x, rows, w, 1e-5), want, atol=1e-12)


@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
def test_a_prefix_has_the_logits_of_the_whole(name, model_root):
    """Nothing looks ahead: the logits of the first tokens do not depend on what follows, across a chunk's edge."""
    folder = make_folder(model_root, name, "float32")
    cfg, w = plain.load_folder(folder)
    tokens = random_tokens(cfg["vocab"], 60, 3)
    whole = plain.forward(cfg, w, tokens)
    assert torch.allclose(plain.forward(cfg, w, tokens[:52]), whole[:52], atol=1e-5)
    layers = []
    plain.forward(cfg, w, tokens[:5], layers_out=layers)
    assert len(layers) == len(cfg["layers"]) and layers[0].shape == (5, cfg["width"])


def test_configuration_round_trip_and_refusals():
    for name, (raw, _, _) in CONFIGS.items():
        cfg = BozasunConfig.from_dict(raw)
        again = BozasunConfig.from_dict(json.loads(json.dumps(cfg.to_dict())))
        assert again == cfg, name
        arch = resolve_architecture(raw)
        model = Model(arch.build_spec(cfg))
        needs = model.tensor_needs()
        assert "head" in needs and "embed" in needs and ("side.embed" in needs) == ("token_side" in raw)
    raw = json.loads(json.dumps(CONFIGS["P"][0]))
    cfg = BozasunConfig.from_dict(raw)
    assert cfg.layers[1].mixer.chunk == 50 and cfg.layers[1].mixer.rot.factor == 5.0 and cfg.layers[0].mlp.identity == 2
    assert cfg.layers[0].mixer.norm_groups == 1 and cfg.side_dim == 5
    needs = Model(resolve_architecture(raw).build_spec(cfg)).tensor_needs()
    assert needs["l0.mlp.router"].shape == (7, 72) and needs["l0.mlp.correction"].shape == (7,)
    assert needs["side.embed"].shape == (200, 4 * 5) and needs["l1.mix.q.b"].shape == (6 * 24,)
    assert needs["l2.mix.g"].shape == (3 * 28, 72) and needs["l0.mix.in"].shape == (2 * 72 + 2 * 10 + 3, 72)
    for change, where in ((lambda r: r["layers"][0].update(type="conv"), "unknown layer type"),
                          (lambda r: r["layers"][1]["mlp"].update(kind="sparse"), "unknown feed-forward kind"),
                          (lambda r: r["layers"][1]["mixer"].update(kv_heads=4), "multiple of kv_heads"),
                          (lambda r: r["layers"][1]["mixer"]["rot"].update(dims=26), "exceeds"),
                          (lambda r: r["layers"][1]["mixer"]["mask"].update(size=0), "positive"),
                          (lambda r: r["layers"][2]["mixer"]["rot"].update(dims=4), "rot_dim"),
                          (lambda r: r["layers"][0]["mlp"]["router"].update(top=9), "experts"),
                          (lambda r: r["layers"][0]["mlp"]["router"].update(groups={"count": 3, "keep": 1}), "groups"),
                          (lambda r: r["layers"][0]["mixer"].update(groups=2), "groups"),
                          (lambda r: r.pop("norm"), "norm")):
        bad = json.loads(json.dumps(raw))
        change(bad)
        with pytest.raises(ConfigError, match=where):
            BozasunConfig.from_dict(bad)


def test_random_model_folder_is_what_the_plain_model_reads(model_root):
    folder = make_folder(model_root, "S", "float32")
    cfg, w = plain.load_folder(folder)
    assert cfg["architecture"] == "Bozasun" and w["l0.mix.q.b"].shape == (2 * 160,) and w["side.embed"].shape == (320, 3)
    assert hb.__name__ and torch.isfinite(plain.forward(cfg, w, random_tokens(320, 12, 1))).all()
