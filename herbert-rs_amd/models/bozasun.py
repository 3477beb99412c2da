"""Bozasun as data: which parts each layer has and what its tensors are called.

A layer is the "prenorm" arrangement, x += mixer(norm1(x)), then, where the layer has a feed-forward,
x += ff(norm2(x)), then, where the model has a table of per-layer token inputs, the part "gated_table" adds to x
from x itself and the tokens' rows of that table; the norms are RMS norms with plain weights. The mixer is

  "attention": the part "attention" with biases, a norm a head whose weights all heads share, a rotation of
      neighbouring pairs whose rates are divided by a constant, the scores' scale a constant of the configuration,
      capped scores, and keys seen only within the query's own chunk of positions;
  "latent_attention": the part "latent_attention" with a gate for every entry of the joined heads and the
      rotation of neighbouring pairs;
  "mamba2": the part "state_space".

The feed-forward is "swiglu" or "routed_experts" whose scores are a softmax over all of the router's outputs, the
last of which stand for experts that are the identity; the choice runs on score + correction within the best
groups (a group being worth its best member), and the weights are the chosen scores as they are. The head is a
matrix of its own. Tensors are stored under short names: `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.<name>`,
`l<i>.mlp.<name>`, `l<i>.side.<name>`, `embed`, `side.embed`, `final.norm`, `head`.
"""
from ..config import register_architecture
from ..config.bozasun import BozasunConfig, DenseConfig
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def _pairs(rot):
    if rot is None:
        return PartSpec("none")
    return PartSpec("rope_pairs", {"theta": rot.base, "rotary_dims": rot.dims,
                                   "scaling": None if rot.factor is None else ("linear", rot.factor)})


def _attention(cfg, m, p):
    names = {k: p + k for k in ("q", "k", "v", "o")}
    names.update(q_norm=p + "q.norm", k_norm=p + "k.norm", q_bias=p + "q.b", k_bias=p + "k.b", v_bias=p + "v.b",
                 o_bias=p + "o.b")
    return PartSpec("attention", {"hidden_size": cfg.hidden_size, "num_heads": m.heads, "num_kv_heads": m.kv_heads,
                                  "head_dim": m.dim, "value_dim": m.vdim, "eps": cfg.norm_eps, "position": _pairs(m.rot),
                                  "names": names, "qk_norm": True, "scale": m.scale, "bias": True, "chunk": m.chunk,
                                  "softcap": m.softcap})


def _latent(cfg, m, p):
    # the angles are computed from the positions, so no table bounds them; the part puts the rotated rows of its
    # projections into the order in which a rotation of halves turns what were neighbours
    scaling = None if m.rot.factor is None else ("linear", m.rot.factor, None, 32.0, 1.0)
    position = PartSpec("rope", {"theta": m.rot.base, "rotary_dims": m.rot.dims,
                                 "max_positions": cfg.max_position_embeddings, "tables": False, "scaling": scaling})
    names = {"q": p + "q", "dkv": p + "dkv", "dkv_norm": p + "dkv.norm", "uk": p + "uk", "uv": p + "uv",
             "g": p + "g", "o": p + "o"}
    return PartSpec("latent_attention", {"hidden_size": cfg.hidden_size, "heads": m.heads, "dim": m.dim,
                                         "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale,
                                         "eps": cfg.norm_eps, "position": position, "names": names,
                                         "gate": "elementwise", "pairs": True})


def _state_space(cfg, m, p):
    names = {"in": p + "in", "conv": p + "conv", "conv_bias": p + "conv.b", "dt_bias": p + "dt_bias",
             "A_log": p + "A_log", "D": p + "D", "norm": p + "norm", "o": p + "o"}
    return PartSpec("state_space", {"hidden_size": cfg.hidden_size, "heads": m.heads, "vdim": m.vdim, "state": m.state,
                                    "groups": m.groups, "conv": m.conv, "eps": cfg.norm_eps, "names": names,
                                    "norm_groups": m.norm_groups})


MIXER_SPECS = {"attention": _attention, "latent_attention": _latent, "mamba2": _state_space}


def _feed_forward(cfg, m, p):
    if isinstance(m, DenseConfig):
        return PartSpec("swiglu", {"hidden_size": cfg.hidden_size, "intermediate_size": m.ff,
                                   "names": {"gate": p + "gate", "up": p + "up", "down": p + "down"}})
    names = {"router": p + "router", "router_bias": p + "correction", "gate": p + "e{e}.gate", "up": p + "e{e}.up",
             "down": p + "e{e}.down"}
    count, keep = m.groups if m.groups is not None else (1, 1)
    return PartSpec("routed_experts", {"hidden_size": cfg.hidden_size, "intermediate_size": m.ff, "experts": m.experts,
                                       "top": m.top, "names": names, "routing": "scores", "scoring": "softmax",
                                       "groups": count, "keep": keep, "group_worth": 1, "renormalize": False,
                                       "activation": "silu", "identity": m.identity})


def _norm(cfg, weight):
    return PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.norm_eps, "weight": weight})


def build_spec(cfg):
    layers = []
    n = len(cfg.layers)
    for i, layer in enumerate(cfg.layers):
        mixer = MIXER_SPECS[layer.type](cfg, layer.mixer, f"l{i}.mix.")
        norms = {"input": _norm(cfg, f"l{i}.norm1")}
        ffn = None
        if layer.mlp is not None:
            ffn = _feed_forward(cfg, layer.mlp, f"l{i}.mlp.")
            norms["post_mixer"] = _norm(cfg, f"l{i}.norm2")
        block = {}
        if cfg.side_dim is not None:
            p = f"l{i}.side."
            block["token_input"] = PartSpec("gated_table", {
                "hidden_size": cfg.hidden_size, "vocab_size": cfg.vocab_size, "dim": cfg.side_dim, "layer": i, "layers": n,
                "eps": cfg.norm_eps, "names": {"table": "side.embed", "gate": p + "gate", "proj": p + "proj", "norm": p + "norm"}})
        layers.append(LayerSpec(PartSpec("prenorm", block), mixer, ffn, norms))
    return ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size, max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("table", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size, "weight": "embed"}),
        layers=layers, schedule=[ScheduleEntry(i) for i in range(n)],
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size, "weight": "head",
                                 "tied_to_embedding": False}),
        eos_token_id=cfg.eos_token_id)


ARCHITECTURE = register_architecture("Bozasun", BozasunConfig, build_spec, model_types=("bozasun",))
