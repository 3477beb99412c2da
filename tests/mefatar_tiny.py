"""Small Mefatar configurations for the tests, their model folders, and the plain logits.

The configurations differ from each other in every size and option: which mixer comes first, keys and values
of different sizes, heads that share keys or not, one head, two to four taps and no filter at all, a rotation
over a part of a head, with and without slowed wavelengths (bands set so that positions of a few hundred
reach all three), blocks of the recurrent unit's gates from one channel to the whole width, layers with and
without a feed-forward, runs of layers repeated two and three times, once, and not at all, constants that are
neither 1 nor equal to each other, and one where they are.
"""
import os

import numpy as np
import torch
from safetensors import safe_open
from safetensors.torch import save_file

import herbert_rs_amd as hb

from .plain import mefatar as plain


def rglru(width, blocks, conv, ff=None):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def rot(dims, base, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return r


def left(heads, kv_heads, dim, vdim, scale, conv, rotation):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if conv is not None:
        m["conv"] = conv
    if rotation is not None:
        m["rot"] = rotation
    return m


def right(heads, dim, vdim, tau, rank):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}


def parallel(l, r, ff=None):
    return {"type": "parallel", "mixer": {"left": l, "right": r}, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def model(vocab, width, layers, eps=1e-5, loop=None):
    raw = {"architecture": "Mefatar", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}}
    if loop is not None:
        raw["loop"] = dict(zip(("start", "stop", "times"), loop))
    return raw


def _p():
    # P: sizes that no kernel's blocks divide; the side-by-side layer first; six heads on two key heads, keys of
    #    24 and values of 40, three taps, 16 of 24 entries rotated with all three bands of wavelengths within
    #    200 positions; layers 1 and 2 three times in a row; a recurrent unit with one block
    layers = [parallel(left(6, 2, 24, 40, 0.3, 3, rot(16, 500.0, (4.0, 1.0, 4.0, 64))), right(3, 24, 40, 7.0, 10), ff=100),
              rglru(96, 3, 4), rglru(40, 1, 2, ff=56)]
    return model(200, 72, layers, eps=3e-6, loop=(1, 3, 3))


def _q():
    # Q: sizes that the matrix cores take as they are (heads of 64, widths in steps of 32); no loop; a unit
    #    without a filter (one tap); two taps on the attention; as many key heads as heads; the whole head rotated
    layers = [rglru(128, 2, 1, ff=256),
              parallel(left(4, 4, 64, 64, 0.125, 2, rot(64, 10000.0)), right(2, 32, 64, 16.0, 16)),
              rglru(192, 6, 3),
              parallel(left(4, 2, 64, 64, 0.2, 4, rot(32, 300.0, (8.0, 1.0, 2.0, 128))), right(4, 32, 32, 4.0, 8), ff=128)]
    return model(384, 128, layers, eps=1e-6)


def _r():
    # R: one head each; no filter on the attention; values wider than a wave, keys of 48 (the matrix cores run
    #    them at 128 with the values); gates of one channel a block; the whole stack twice
    layers = [parallel(left(1, 1, 48, 80, 0.06, None, rot(48, 50.0)), right(1, 16, 80, 1.0, 5), ff=24),
              rglru(32, 32, 4)]
    return model(96, 64, layers, eps=1e-5, loop=(0, 2, 2))


def _s():
    # S: heads beyond 128 (the plain attention kernel in either mode), the side-by-side layer alone looped, a
    #    loop that runs once, keys of the linear attention that four does not divide
    layers = [rglru(80, 5, 2),
              parallel(left(2, 1, 160, 144, 0.08, 2, rot(6, 20.0, (2.0, 0.5, 3.0, 32))), right(2, 22, 48, 3.0, 12), ff=96),
              parallel(left(6, 3, 32, 16, 0.2, 4, None), right(3, 40, 24, 30.0, 20))]
    return model(320, 192, layers, eps=2e-5, loop=(1, 2, 1))


def _w():
    # W: the widths of a larger model's layers at a small depth: heads of 128, a unit wider than the model
    layers = [parallel(left(8, 2, 128, 128, 0.09, 4, rot(128, 10000.0, (8.0, 1.0, 4.0, 256))), right(4, 64, 128, 16.0, 32), ff=1024),
              rglru(768, 6, 4)]
    return model(1024, 512, layers, eps=1e-6, loop=(0, 2, 2))


def _f():
    # F: for keys far back and long memories: scores three times as sharp as a random model's usual ones (the
    #    scale), and the tests set the decays of both recurrences near one
    layers = [rglru(128, 4, 3),
              parallel(left(4, 2, 64, 64, 0.4, 3, rot(64, 1000.0, (4.0, 1.0, 4.0, 128))), right(2, 32, 32, 8.0, 16), ff=256)]
    return model(384, 128, layers, eps=1e-6, loop=(0, 2, 2))


CONFIGS = {"F": (_f(), 36, 0.09), "P": (_p(), 31, 0.12), "Q": (_q(), 32, 0.09), "R": (_r(), 33, 0.15), "S": (_s(), 34, 0.08),
           "W": (_w(), 35, 0.05)}


def make_folder(root, name, dtype="float32", scale=None, set_to=None, tag=""):
    """Write the random model `name` into root/<name>_<dtype><tag> once. `scale` {tensor name suffix: factor}
    multiplies tensors afterwards, `set_to` {suffix: value} fills them: to make a far key, a sink or a long
    memory show where random weights would hide it."""
    raw, seed, std = CONFIGS[name]
    folder = os.path.join(str(root), f"mef_{name}_{dtype}{tag}")
    if os.path.exists(os.path.join(folder, "model.safetensors")):
        return folder
    hb.write_random_model(folder, raw, seed=seed, dtype=dtype, std=std, norm_std=0.1)
    if scale or set_to:
        path = os.path.join(folder, "model.safetensors")
        tensors = {}
        with safe_open(path, framework="pt") as f:
            for k in f.keys():
                tensors[k] = f.get_tensor(k)
        for k in tensors:
            for suffix, factor in (scale or {}).items():
                if k.endswith(suffix):
                    tensors[k] = (tensors[k].float() * factor).to(tensors[k].dtype)
            for suffix, value in (set_to or {}).items():
                if k.endswith(suffix):
                    tensors[k] = torch.full_like(tensors[k], value)
        save_file(tensors, path)
    return folder


_folders, _logits = {}, {}


def plain_folder(folder):
    if folder not in _folders:
        _folders[folder] = plain.load_folder(folder)
    return _folders[folder]


def plain_logits(folder, tokens):
    """float32 [len(tokens), vocab] of the plain whole-sequence implementation, computed once."""
    key = (folder, tuple(tokens))
    if key not in _logits:
        cfg, w = plain_folder(folder)
        _logits[key] = plain.forward(cfg, w, list(tokens)).numpy().astype(np.float32)
    return _logits[key]


def random_tokens(vocab, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
