"""Small Bozasun configurations for the tests, their model folders, and the plain logits.

The configurations differ from each other in every size and option: which mixer comes first and last, keys and
values of different sizes, heads that share keys or not, one head, chunks of positions shorter than a page, a
page's multiple, neither, and none at all, capped scores or not, a rotation over a part of a head or the whole of
it, slowed or not, latents and rotated parts that the matrix cores take and that they do not, state-space layers
with one group and several, one tap to four, one norm group and several, experts in groups and not, with and
without identity experts, every expert chosen, layers without a feed-forward, models with and without the
per-layer token input, constants that are neither 1 nor equal to each other.
"""
import os

import numpy as np
import torch
from safetensors import safe_open
from safetensors.torch import save_file

import herbert_rs_amd as hb

from .plain import bozasun as plain


def rot(dims, base, factor=None):
    r = {"dims": dims, "base": base}
    if factor is not None:
        r["scaling"] = {"factor": factor}
    return r


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, identity=0, groups=None):
    router = {"experts": experts, "top": top}
    if identity:
        router["identity"] = identity
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def attention(heads, kv_heads, dim, vdim, scale, rotation=None, chunk=None, softcap=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rotation is not None:
        m["rot"] = rotation
    if chunk is not None:
        m["mask"] = {"size": chunk}
    if softcap is not None:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base, mlp=None, factor=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": rot(rot_dim, base, factor)}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def mamba(heads, vdim, state, groups, conv, norm_groups=None, mlp=None):
    m = {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv}
    if norm_groups is not None:
        m["norm_groups"] = norm_groups
    return {"type": "mamba2", "mixer": m, "mlp": mlp}


def model(vocab, width, layers, eps=1e-5, side=None):
    raw = {"architecture": "Bozasun", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}}
    if side is not None:
        raw["token_side"] = {"dim": side}
    return raw


def _p():
    # P: sizes that no kernel's blocks divide; the state-space layer first; chunks of 50 positions (neither a page
    #    nor a part of one); six heads on two key heads, keys of 24 and values of 40, 16 of 24 entries rotated at
    #    a fifth of the rate; five experts and two identity experts, no groups; a latent of 40 + 6
    layers = [mamba(3, 24, 10, 1, 3, mlp=moe(36, 5, 2, identity=2)),
              attention(6, 2, 24, 40, 0.3, rot(16, 500.0, 5.0), chunk=50, softcap=8.0, mlp=dense(100)),
              latent(3, 20, 6, 28, 40, 0.2, 300.0, mlp=moe(36, 5, 2, identity=2)),
              attention(6, 2, 24, 40, 0.3, rot(16, 500.0, 5.0), chunk=50, softcap=8.0)]
    return model(200, 72, layers, eps=3e-6, side=5)


def _q():
    # Q: sizes that the matrix cores take as they are (heads of 64, widths in steps of 32, a latent of 64 + 32);
    #    chunks of 128 (two pages); as many key heads as heads; the whole head rotated, not slowed; no cap on one
    #    attention layer; experts in four groups of which two count, no identity experts; four taps, two groups
    #    of B and C, four norm groups
    layers = [attention(4, 4, 64, 64, 0.125, rot(64, 10000.0), chunk=128, mlp=moe(64, 8, 2, groups=(4, 2))),
              mamba(4, 32, 16, 2, 4, norm_groups=4, mlp=dense(256)),
              latent(4, 32, 32, 64, 64, 0.15, 10000.0, mlp=dense(128)),
              attention(4, 2, 64, 64, 0.2, rot(32, 300.0, 2.0), chunk=128, softcap=20.0, mlp=moe(64, 6, 3, identity=2, groups=(4, 3)))]
    return model(384, 128, layers, eps=1e-6, side=32)


def _r():
    # R: one head each; no chunks (every earlier key is seen) and no rotation on one layer; values wider than a
    #    wave, keys of 48; a state of 40 rows and one tap (no filter); every expert chosen; no token input
    layers = [latent(1, 16, 4, 80, 24, 0.3, 50.0, mlp=moe(24, 3, 3)),
              attention(1, 1, 48, 80, 0.06, None, softcap=3.0, mlp=dense(24)),
              mamba(1, 80, 40, 1, 1, mlp=None),
              attention(1, 1, 48, 80, 0.06, rot(48, 50.0), mlp=moe(24, 2, 3, identity=1))]
    return model(96, 64, layers, eps=1e-5)


def _s():
    # S: heads beyond 128 (the plain attention kernel in either mode); chunks of 7 positions; a token input as
    #    wide as 1; groups of experts that hold one expert each; a layer without a feed-forward; a latent beyond
    #    what the matrix cores take in one piece (rank 72)
    layers = [attention(2, 1, 160, 144, 0.08, rot(6, 20.0, 3.0), chunk=7, softcap=50.0, mlp=moe(40, 4, 2, identity=2, groups=(6, 3))),
              mamba(6, 16, 64, 3, 2, norm_groups=2, mlp=None),
              latent(2, 40, 8, 24, 72, 0.1, 1000.0, mlp=dense(96))]
    return model(320, 192, layers, eps=2e-5, side=1)


def _w():
    # W: the widths of a larger model's layers at a small depth: heads of 128, a state of 128 rows and columns of 64
    layers = [attention(8, 2, 128, 128, 0.09, rot(128, 250000.0, 4.0), chunk=192, softcap=25.0, mlp=moe(256, 8, 2, identity=2, groups=(5, 2))),
              mamba(8, 64, 128, 2, 4, norm_groups=2, mlp=dense(1024)),
              latent(8, 64, 32, 64, 256, 0.1, 10000.0, mlp=moe(256, 8, 2, identity=2, groups=(5, 2)))]
    return model(1024, 512, layers, eps=1e-6, side=64)


def _f():
    # F: for keys far back and long memories: scores twice as sharp as a random model's usual ones (the
    #    scale), no chunks on the first attention so that it sees the whole sequence, chunks of 64 on the second;
    #    the tests set the state-space layer's decay near one
    layers = [attention(4, 2, 64, 64, 0.25, rot(64, 1000.0, 4.0), softcap=40.0, mlp=dense(256)),
              mamba(4, 32, 32, 2, 3, mlp=dense(128)),
              latent(4, 32, 32, 32, 64, 0.25, 1000.0, mlp=dense(128)),
              attention(4, 2, 64, 64, 0.25, rot(64, 1000.0, 4.0), chunk=64, softcap=40.0, mlp=dense(256))]
    return model(384, 128, layers, eps=1e-6, side=8)


CONFIGS = {"F": (_f(), 46, 0.09), "P": (_p(), 41, 0.12), "Q": (_q(), 42, 0.09), "R": (_r(), 43, 0.15), "S": (_s(), 44, 0.08),
           "W": (_w(), 45, 0.05)}


def make_folder(root, name, dtype="float32", scale=None, set_to=None, tag=""):
    """Write the random model `name` into root/<name>_<dtype><tag> once. `scale` {tensor name suffix: factor}
    multiplies tensors afterwards, `set_to` {suffix: value} fills them: to make a far key, a chunk's edge or a long
    memory show where random weights would hide it."""
    raw, seed, std = CONFIGS[name]
    folder = os.path.join(str(root), f"boz_{name}_{dtype}{tag}")
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
