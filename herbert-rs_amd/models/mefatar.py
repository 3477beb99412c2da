"""Mefatar as data: which parts each layer has and what its tensors are called.

A layer is the "prenorm" arrangement with scaled branches: x += ls1 * mixer(norm1(x)), then, where the layer
has a feed-forward, x += ls2 * ff(norm2(x)); the norms are RMS norms with plain weights. The mixer is a
real-gated linear recurrent unit ("rglru": the part "gated_lru") or two mixers side by side on the same rows
("parallel": the part "side_by_side" of an "attention" with a filter, a norm over the whole projection, a
rotation of pairs with scaled rates, a sink and a gate, and a "decayed_linear_attention"), whose outputs are
normed over the model's width and averaged. The feed-forward is the gated unit with the tanh form of gelu. A
run of adjacent layers may be repeated: every pass is a further entry of the schedule on the same layer, with
a cache and states of its own. The logits are the table itself times the normed last rows. Tensors are stored
under short names: `l<i>.norm1`, `l<i>.norm2`, `l<i>.ls1`, `l<i>.ls2`, `l<i>.mix.<name>`, `l<i>.mlp.<name>`,
`embed`, `final.norm`.
"""
from ..config import register_architecture
from ..config.mefatar import MefatarConfig
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

LRU_RATE = 8.0          # the recurrent unit's decay is exp(-8 r softplus(lam)) in every model of the design


def _recurrent(cfg, m, p):
    names = {"x": p + "x", "x_bias": p + "x.b", "y": p + "y", "y_bias": p + "y.b", "conv": p + "conv",
             "conv_bias": p + "conv.b", "r": p + "ra", "r_bias": p + "ra.b", "i": p + "ri", "i_bias": p + "ri.b",
             "lam": p + "lam", "o": p + "o"}
    return PartSpec("gated_lru", {"hidden_size": cfg.hidden_size, "width": m.width, "blocks": m.blocks, "conv": m.conv,
                                  "names": names, "rate": LRU_RATE})


def _left(cfg, m, p):
    names = {k: p + k for k in ("q", "k", "v", "o", "g", "sink")}
    names.update(q_norm=p + "q.norm", k_norm=p + "k.norm", q_conv=p + "q.conv", k_conv=p + "k.conv", v_conv=p + "v.conv")
    position = PartSpec("none")
    if m.rot is not None:
        sc = m.rot.scaling
        position = PartSpec("rope_pairs", {"theta": m.rot.base, "rotary_dims": m.rot.dims,
                                           "scaling": None if sc is None else (sc.factor, sc.low, sc.high, sc.original)})
    return PartSpec("attention", {"hidden_size": cfg.hidden_size, "num_heads": m.heads, "num_kv_heads": m.kv_heads,
                                  "head_dim": m.dim, "value_dim": m.vdim, "eps": cfg.norm_eps, "position": position,
                                  "names": names, "qk_norm": "whole", "scale": m.scale, "conv": m.conv, "sink": True,
                                  "gate": True})


def _right(cfg, m, p):
    names = {k: p + k for k in ("q", "k", "v", "g", "a1", "a2", "norm", "o")}
    names["a2_bias"] = p + "a2.b"
    return PartSpec("decayed_linear_attention", {"hidden_size": cfg.hidden_size, "heads": m.heads, "dim": m.dim,
                                                 "vdim": m.vdim, "tau": m.tau, "eps": cfg.norm_eps, "names": names,
                                                 "rank": m.rank})


def _parallel(cfg, m, p):
    return PartSpec("side_by_side", {"hidden_size": cfg.hidden_size, "left": _left(cfg, m.left, p + "left."),
                                     "right": _right(cfg, m.right, p + "right."), "eps": cfg.norm_eps,
                                     "names": {"left_norm": p + "left.out", "right_norm": p + "right.out"},
                                     "weights": (0.5, 0.5)})


MIXER_SPECS = {"rglru": _recurrent, "parallel": _parallel}


def _norm(cfg, weight):
    return PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.norm_eps, "weight": weight})


def build_spec(cfg):
    layers = []
    for i, layer in enumerate(cfg.layers):
        mixer = MIXER_SPECS[layer.type](cfg, layer.mixer, f"l{i}.mix.")
        norms = {"input": _norm(cfg, f"l{i}.norm1")}
        scale = {"size": cfg.hidden_size, "mixer": f"l{i}.ls1"}
        ffn = None
        if layer.mlp is not None:
            p = f"l{i}.mlp."
            ffn = PartSpec("swiglu", {"hidden_size": cfg.hidden_size, "intermediate_size": layer.mlp.ff,
                                      "names": {"gate": p + "gate", "up": p + "up", "down": p + "down"},
                                      "activation": "gelu_tanh"})
            norms["post_mixer"] = _norm(cfg, f"l{i}.norm2")
            scale["feed_forward"] = f"l{i}.ls2"
        layers.append(LayerSpec(PartSpec("prenorm", {"branch_scale": scale}), mixer, ffn, norms))
    # every run of a layer is an entry of the schedule with a cache and states of its own, whichever pass it is
    schedule = [ScheduleEntry(i) for i in cfg.layer_runs()]
    return ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size, max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("table", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size, "weight": "embed"}),
        layers=layers, schedule=schedule,
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size, "weight": "embed",
                                 "tied_to_embedding": True}),
        eos_token_id=cfg.eos_token_id)


ARCHITECTURE = register_architecture("Mefatar", MefatarConfig, build_spec, model_types=("mefatar",))
