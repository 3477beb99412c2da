"""Plain, slow, whole-sequence formulas of the Bozasun decoder: one function a mechanism.

A model of this design is a stack of pre-norm layers

    x <- x + mixer(norm1(x));  x <- x + ff(norm2(x));  x <- x + side(x, token)

with norm(x) = x / sqrt(mean(x^2) + eps) * w. The second step is there where the layer has a feed-forward, the
third where the model has a table of per-layer token inputs. A mixer is a softmax attention over the keys of
the query's own chunk of positions, with biases, a norm a head, a rotation of neighbouring pairs at slowed
rates and capped scores ("attention"); an attention whose keys and values all come from one low-rank latent
a token and a small rotated part that every head shares, with a gate on the joined heads
("latent_attention"); or a state-space layer with one decay a head ("mamba2"). The feed-forward is a gated
unit or a mixture of such units among which some "experts" are the identity. Nothing here has a cache, a
batch or code in common with the engine; everything runs on the CPU in the dtype of its inputs (float32, or
float64 to judge rounding).
"""
import json
import math
import os

import torch
from safetensors import safe_open


# ---------------------------------------------------------------- small pieces
def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis (w None: no weight)."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def linear(x, weight, bias=None):
    y = x @ weight.T
    return y if bias is None else y + bias


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.minimum(x, torch.full_like(x, 30.0)))))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z * z * z)))


# ---------------------------------------------------------------- rotation
def pair_rates(rot):
    """The angle a position of pair i: base^(-2i / dims), every rate divided by the scaling's factor."""
    dims = rot["dims"]
    f = torch.tensor([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    sc = rot.get("scaling")
    if sc is not None:
        f = f / sc["factor"]
    return f


def rotate_pairs(x, positions, rot):
    """x [T, heads, D]: entries 2i and 2i + 1 of the first rot.dims turn by position x rate_i; the rest stay."""
    if rot is None:
        return x
    dims = rot["dims"]
    ang = positions.to(torch.float64)[:, None] * pair_rates(rot)[None, :]          # [T, dims / 2]
    cos, sin = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ---------------------------------------------------------------- attention over chunks
def visible(positions, chunk):
    """[T, T] True where the key at column j is seen by the query at row i: j <= i, and with chunks only
    within the same chunk of `chunk` positions counted from the start of the sequence."""
    i, j = positions[:, None], positions[None, :]
    see = j <= i
    if chunk:
        see = see & (torch.div(i, chunk, rounding_mode="floor") == torch.div(j, chunk, rounding_mode="floor"))
    return see


def masked_softmax_attention(q, k, v, see, scale, softcap=None):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; query head h reads key head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~see, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, h] = p @ v[:, g]
    return out


def attention_mixer(h, w, m, eps, positions):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w["q"], w["q.b"]).view(T, H, D)
    k = linear(h, w["k"], w["k.b"]).view(T, G, D)
    v = linear(h, w["v"], w["v.b"]).view(T, G, Dv)
    q = rms_norm(q, w["q.norm"], eps)
    k = rms_norm(k, w["k.norm"], eps)
    q = rotate_pairs(q, positions, m.get("rot"))
    k = rotate_pairs(k, positions, m.get("rot"))
    chunk = (m.get("mask") or {}).get("size")
    o = masked_softmax_attention(q, k, v, visible(positions, chunk), m["scale"], m.get("softcap"))
    return linear(o.reshape(T, H * Dv), w["o"], w["o.b"])


# ---------------------------------------------------------------- latent attention
def latent_attention_mixer(h, w, m, eps, positions):
    T = h.shape[0]
    H, D, R, Dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = dict(m["rot"])
    q = linear(h, w["q"]).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], rotate_pairs(q[..., D:].contiguous(), positions, rot)
    down = linear(h, w["dkv"])
    c = rms_norm(down[:, :rank], w["dkv.norm"], eps)
    k_rot = rotate_pairs(down[:, None, rank:].contiguous(), positions, rot)[:, 0]          # [T, R], one for all heads
    k_plain = linear(c, w["uk"]).view(T, H, D)
    v = linear(c, w["uv"]).view(T, H, Dv)
    see = visible(positions, None)
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * m["scale"]
        s = s.masked_fill(~see, float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, a]
    gated = out.reshape(T, H * Dv) * sigmoid(linear(h, w["g"]))
    return linear(gated, w["o"])


# ---------------------------------------------------------------- state-space layer
def causal_taps(u, taps, bias):
    """u [T, C], taps [C, K]: y_t = bias + sum_j taps[:, j] u_(t - K + 1 + j), nothing before the first row."""
    T, K = u.shape[0], taps.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(K):
            s = t - K + 1 + j
            if s >= 0:
                y[t] += taps[:, j] * u[s]
    return y + bias


def state_space_walk(x, B, C, dt, a_log, d_skip):
    """x [T, H, P], B and C [T, G, N], dt [T, H] (after its softplus): a matrix [N, P] a head,
    S <- exp(-exp(a_log) dt) S + dt B x^T, y = S^T C + d_skip x."""
    T, H, P = x.shape
    G, N = B.shape[1], B.shape[2]
    y = torch.zeros_like(x)
    for a in range(H):
        g = a // (H // G)
        S = torch.zeros(N, P, dtype=x.dtype)
        rate = torch.exp(a_log[a])
        for t in range(T):
            S = torch.exp(-rate * dt[t, a]) * S + dt[t, a] * torch.outer(B[t, g], x[t, a])
            y[t, a] = S.T @ C[t, g] + d_skip[a] * x[t, a]
    return y


def mamba2_mixer(h, w, m, eps):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = linear(h, w["in"])
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_taps(xbc, w["conv"], w["conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w["dt_bias"])
    y = state_space_walk(x, B, C, dt, w["A_log"], w["D"]).reshape(T, inner)
    y = y * silu(z)
    parts = m.get("norm_groups", 1)
    y = rms_norm(y.view(T, parts, inner // parts), None, eps).reshape(T, inner) * w["norm"]
    return linear(y, w["o"])


# ---------------------------------------------------------------- feed-forward
def gated_unit(h, gate, up, down):
    return linear(silu(linear(h, gate)) * linear(h, up), down)


def choose_experts(scores, correction, top, groups):
    """scores [E] -> the indices of the `top` largest of scores + correction, the lower index of equals first;
    with groups = (count, keep) only among the `keep` runs of E / count neighbours whose largest such value is
    largest."""
    choice = scores + correction
    E = choice.shape[0]
    allowed = torch.ones(E, dtype=torch.bool)
    if groups is not None:
        count, keep = groups
        per = E // count
        worth = choice.view(count, per).max(dim=1).values
        order = sorted(range(count), key=lambda g: (-worth[g].item(), g))[:keep]
        allowed = torch.zeros(E, dtype=torch.bool)
        for g in order:
            allowed[g * per:(g + 1) * per] = True
    ranked = sorted((e for e in range(E) if allowed[e]), key=lambda e: (-choice[e].item(), e))
    return ranked[:top]


def moe_ff(h, w, mlp):
    r = mlp["router"]
    real, ident = r["experts"], r.get("identity", 0)
    groups = None if r.get("groups") is None else (r["groups"]["count"], r["groups"]["keep"])
    scores = torch.softmax(linear(h, w["router"]), dim=-1)          # over experts and identity experts together
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in choose_experts(scores[t], w["correction"], r["top"], groups):
            if e < real:
                y = gated_unit(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])[0]
            else:
                y = h[t]
            out[t] += scores[t, e] * y
    return out


def feed_forward(h, w, mlp):
    if mlp["kind"] == "dense":
        return gated_unit(h, w["gate"], w["up"], w["down"])
    return moe_ff(h, w, mlp)


# ---------------------------------------------------------------- per-layer token input
def token_side(x, rows, w, eps):
    """rows [T, dim]: this layer's part of the tokens' side table. x + norm(W_proj (gelu(W_gate x) * rows))."""
    y = linear(gelu_tanh(linear(x, w["gate"])) * rows, w["proj"])
    return x + rms_norm(y, w["norm"], eps)


# ---------------------------------------------------------------- the model
def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens, dtype=torch.float32, layers_out=None, rows=None):
    """Logits [T, vocab] (or at `rows`) of one sequence from its first token on."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.shape[0])
    x = w["embed"][tokens]
    side = cfg.get("token_side")
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_norm(x, w[p + "norm1"], eps)
        mw = sub(w, p + "mix.")
        if layer["type"] == "attention":
            x = x + attention_mixer(h, mw, layer["mixer"], eps, positions)
        elif layer["type"] == "latent_attention":
            x = x + latent_attention_mixer(h, mw, layer["mixer"], eps, positions)
        elif layer["type"] == "mamba2":
            x = x + mamba2_mixer(h, mw, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            x = x + feed_forward(rms_norm(x, w[p + "norm2"], eps), sub(w, p + "mlp."), layer["mlp"])
        if side is not None:
            d = side["dim"]
            x = token_side(x, w["side.embed"][tokens][:, i * d:(i + 1) * d], sub(w, p + "side."), eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms_norm(x, w["final.norm"], eps)
    if rows is not None:
        x = x[torch.as_tensor(rows, dtype=torch.long)]
    return linear(x, w["head"])


def greedy(cfg, tensors, prompt, n):
    """The n tokens that follow `prompt` when the most likely one (the lower of equals) is taken each time."""
    tokens = list(prompt)
    out = []
    for _ in range(n):
        logits = forward(cfg, tensors, tokens, rows=[len(tokens) - 1])[0]
        out.append(int(torch.argmax(logits)))
        tokens.append(out[-1])
    return out


def load_folder(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        for k in f.keys():
            tensors[k] = f.get_tensor(k)
    return cfg, tensors
