"""Plain, slow, whole-sequence formulas of the Mefatar decoder: one function a mechanism.

A model of this design is a stack of pre-norm layers with a learned scale a channel on every branch:

    x <- x + ls1 * mixer(norm1(x));  x <- x + ls2 * ff(norm2(x))      (the second step only where the layer has a feed-forward)

with norm(x) = x / sqrt(mean(x^2) + eps) * w. A mixer is a real-gated linear recurrent unit between two
branches ("rglru"), or two mixers side by side on the same input ("parallel"): a softmax attention whose
queries, keys and values pass a short filter along time, whose queries and keys are normed over the
whole projection and rotated pair by pair, and whose softmax has a sink; and a linear attention whose
state decays channel by channel. Their outputs are each normed over the model's width and averaged. A run
of adjacent layers may be repeated, every pass with states of its own. Nothing here has a cache, a batch or
code in common with the engine; everything runs on the CPU in the dtype of its inputs (float32, or
float64 to judge rounding).
"""
import json
import math
import os

import torch
from safetensors import safe_open

LRU_RATE = 8.0          # the recurrent unit's decay is exp(-LRU_RATE * gate * softplus(lam))


# ---------------------------------------------------------------- small pieces
def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def linear(x, weight, bias=None):
    y = x @ weight.T
    return y if bias is None else y + bias


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 20.0, x, torch.log1p(torch.exp(torch.minimum(x, torch.full_like(x, 20.0)))))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z * z * z)))


def causal_filter(u, taps, bias=None):
    """u [T, C], taps [C, K]: y_t = sum_j taps[:, j] * u_(t - K + 1 + j), nothing before the first row."""
    T, K = u.shape[0], taps.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(K):
            s = t - K + 1 + j
            if s >= 0:
                y[t] += taps[:, j] * u[s]
    return y if bias is None else y + bias


# ---------------------------------------------------------------- rotation
def rotation_rates(rot, dtype=torch.float64):
    """The angle a position of pair i: base^(-2i / dims), and where `scaling` is given, long wavelengths
    slowed down: those beyond original / low by `factor`, those under original / high not at all, a blend
    between."""
    dims = rot["dims"]
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = rot["base"] ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if sc is not None:
        factor, low, high, original = sc["factor"], sc["low"], sc["high"], sc["original"]
        out = f.clone()
        for n in range(f.shape[0]):
            wavelength = 2.0 * math.pi / f[n].item()
            if wavelength < original / high:
                continue
            if wavelength > original / low:
                out[n] = f[n] / factor
            else:
                s = (original / wavelength - low) / (high - low)
                out[n] = (1.0 - s) * f[n] / factor + s * f[n]
        f = out
    return f.to(dtype)


def rotate_pairs(x, positions, rates, dims):
    """x [T, heads, D]: entries 2i and 2i + 1 of the first `dims` turn by positions * rates[i]."""
    out = x.clone()
    angle = positions.to(rates.dtype)[:, None] * rates[None, :]           # [T, dims / 2]
    cos, sin = torch.cos(angle).to(x.dtype)[:, None, :], torch.sin(angle).to(x.dtype)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


# ---------------------------------------------------------------- softmax attention with a sink
def sink_attention(q, k, v, scale, sink):
    """One head over T tokens, causal: row i sees rows 0 .. i; the softmax's denominator also holds
    exp(sink), which has no key and no value. q, k [T, D]; v [T, V]; sink a number."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=q.dtype)
    for i in range(T):
        s = (k[: i + 1] @ q[i]) * scale
        m = torch.maximum(s.max(), sink)
        p = torch.exp(s - m)
        out[i] = (p / (p.sum() + torch.exp(sink - m))) @ v[: i + 1]
    return out


def left_mixer(h, w, m, eps, positions=None):
    """h [T, W]; w: q, k, v, (q.conv, k.conv, v.conv,) q.norm, k.norm, sink, g, o; m: heads, kv_heads, dim,
    vdim, conv, rot {dims, base, scaling}, scale."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = linear(h, w["q"]), linear(h, w["k"]), linear(h, w["v"])
    if m.get("conv"):
        q, k, v = causal_filter(q, w["q.conv"]), causal_filter(k, w["k.conv"]), causal_filter(v, w["v.conv"])
    q = rms_norm(q, w["q.norm"], eps).view(T, H, D)
    k = rms_norm(k, w["k.norm"], eps).view(T, G, D)
    v = v.view(T, G, V)
    rot = m.get("rot")
    if rot is not None:
        pos = torch.arange(T) if positions is None else positions
        rates = rotation_rates(rot)
        q, k = rotate_pairs(q, pos, rates, rot["dims"]), rotate_pairs(k, pos, rates, rot["dims"])
    heads = [sink_attention(q[:, i], k[:, i // (H // G)], v[:, i // (H // G)], m["scale"], w["sink"][i]) for i in range(H)]
    o = torch.stack(heads, 1).reshape(T, H * V)
    return linear(o * sigmoid(linear(h, w["g"])), w["o"])


# ---------------------------------------------------------------- linear attention with a decay a key channel
def decaying_state_attention(q, k, v, alpha):
    """One head: S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t. q, k, alpha [T, D]; v [T, V]."""
    T, D = q.shape
    S = torch.zeros(D, v.shape[1], dtype=q.dtype)
    out = torch.zeros(T, v.shape[1], dtype=q.dtype)
    for t in range(T):
        S = alpha[t][:, None] * S + torch.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out


def right_mixer(h, w, m, eps):
    """w: q, k, v, a1, a2, a2.b, norm, g, o; m: heads, dim, vdim, tau."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (linear(h, w["q"]) * D ** -0.5).view(T, H, D)
    k = linear(h, w["k"]).view(T, H, D)
    v = linear(h, w["v"]).view(T, H, V)
    z = linear(linear(h, w["a1"]), w["a2"], w["a2.b"])
    alpha = (sigmoid(z) ** (1.0 / m["tau"])).view(T, H, D)
    o = torch.stack([decaying_state_attention(q[:, i], k[:, i], v[:, i], alpha[:, i]) for i in range(H)], 1)
    o = rms_norm(o, w["norm"], eps).reshape(T, H * V)
    return linear(o * silu(linear(h, w["g"])), w["o"])


def parallel_mixer(h, w, m, eps, positions=None):
    left = left_mixer(h, sub(w, "left."), m["left"], eps, positions)
    right = right_mixer(h, sub(w, "right."), m["right"], eps)
    return 0.5 * (rms_norm(left, w["left.out"], eps) + rms_norm(right, w["right.out"], eps))


# ---------------------------------------------------------------- real-gated linear recurrent unit
def gated_recurrence(u, r, i, lam):
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t with a_t = exp(-LRU_RATE r_t softplus(lam)), S = 0 before the
    first token. u, r, i [T, C]; lam [C]."""
    S = torch.zeros_like(u[0])
    out = torch.zeros_like(u)
    for t in range(u.shape[0]):
        a = torch.exp(-LRU_RATE * r[t] * softplus(lam))
        S = a * S + torch.sqrt(1.0 - a * a) * i[t] * u[t]
        out[t] = S
    return out


def block_product(u, mats, bias):
    """u [T, blocks x n] through a square matrix [out, in] a block: mats [blocks, n, n], bias [blocks, n]."""
    B, n = mats.shape[0], mats.shape[1]
    parts = [u[:, b * n:(b + 1) * n] @ mats[b].T + bias[b] for b in range(B)]
    return torch.cat(parts, -1)


def rglru_mixer(h, w, m):
    """w: y, y.b, x, x.b, conv, conv.b, ra, ra.b, ri, ri.b, lam, o; m: width, blocks, conv."""
    y = gelu_tanh(linear(h, w["y"], w["y.b"]))
    u = causal_filter(linear(h, w["x"], w["x.b"]), w["conv"], w["conv.b"])
    r = sigmoid(block_product(u, w["ra"], w["ra.b"]))
    i = sigmoid(block_product(u, w["ri"], w["ri.b"]))
    return linear(gated_recurrence(u, r, i, w["lam"]) * y, w["o"])


# ---------------------------------------------------------------- feed-forward
def dense_ff(h, w):
    return linear(gelu_tanh(linear(h, w["gate"])) * linear(h, w["up"]), w["down"])


# ---------------------------------------------------------------- the model
def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def layer_runs(cfg):
    """The layers in the order they run: layers start .. stop - 1 `times` times in a row, the rest once."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if loop is None:
        return list(range(n))
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def forward(cfg, tensors, tokens, dtype=torch.float32, layers_out=None, rows=None):
    """Logits [T, vocab] of one sequence of token ids (of the positions `rows` only, if given).
    layers_out: a list that receives the residual stream after every layer run."""
    t = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i in layer_runs(cfg):
        layer, p = cfg["layers"][i], f"l{i}."
        h = rms_norm(x, t[p + "norm1"], eps)
        if layer["type"] == "rglru":
            mixed = rglru_mixer(h, sub(t, p + "mix."), layer["mixer"])
        elif layer["type"] == "parallel":
            mixed = parallel_mixer(h, sub(t, p + "mix."), layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + t[p + "ls1"] * mixed
        if layer.get("mlp") is not None:
            x = x + t[p + "ls2"] * dense_ff(rms_norm(x, t[p + "norm2"], eps), sub(t, p + "mlp."))
        if layers_out is not None:
            layers_out.append(x.clone())
    if rows is not None:
        x = x[list(rows)]
    return linear(rms_norm(x, t["final.norm"], eps), t["embed"])


def greedy(cfg, tensors, prompt, n):
    """n tokens after the prompt, each the first of the largest logits of the sequence so far."""
    seq, out = list(prompt), []
    for _ in range(n):
        logits = forward(cfg, tensors, seq, rows=[len(seq) - 1])[0]
        out.append(int(torch.argmax(logits)))
        seq.append(out[-1])
    return out


def load_folder(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name)
    return cfg, tensors
