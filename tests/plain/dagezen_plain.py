"""Dagezen written plainly: float64 numpy, one function per mechanism, token by token where a mechanism is
sequential.  It shares nothing with the library: the tests hold the library to it.

``weights`` maps checkpoint names to float64 arrays, ``cfg`` is the dictionary of config.json.
"""
from __future__ import annotations

import math

import numpy as np


def gelu_erf(z):
    return 0.5 * z * (1.0 + np.vectorize(math.erf)(z / math.sqrt(2.0)))


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * w + b


def rotate_pairs(x, positions, dims, base):
    """x [T, heads, dim]: the neighbours (2i, 2i + 1) of the first ``dims`` elements of every head turn by
    positions * base^(-2i / dims); the rest stays."""
    out = x.copy()
    for i in range(dims // 2):
        a = positions * base ** (-2.0 * i / dims)
        c, s = np.cos(a)[:, None], np.sin(a)[:, None]
        u, v = x[:, :, 2 * i], x[:, :, 2 * i + 1]
        out[:, :, 2 * i] = u * c - v * s
        out[:, :, 2 * i + 1] = v * c + u * s
    return out


# ---------------------------------------------------------------- latent attention
def latent_mixer(h, w, p, m, eps, state):
    t = h.shape[0]
    heads, dim, rot, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    start = state.get("len", 0)
    pos = np.arange(start, start + t, dtype=np.float64)
    q = (h @ w[p + "q"].T).reshape(t, heads, dim + rot)
    q_plain, q_rot = q[:, :, :dim], rotate_pairs(q[:, :, dim:], pos, m["rot"]["dims"], m["rot"]["base"])
    dkv = h @ w[p + "dkv"].T
    c = rms_unit(dkv[:, :rank], eps) * w[p + "dkv.norm"]
    k_rot = rotate_pairs(dkv[:, None, rank:], pos, m["rot"]["dims"], m["rot"]["base"])[:, 0]
    state["c"] = np.concatenate([state["c"], c]) if "c" in state else c
    state["kr"] = np.concatenate([state["kr"], k_rot]) if "kr" in state else k_rot
    state["len"] = start + t
    all_c, all_kr = state["c"], state["kr"]
    k_plain = (all_c @ w[p + "uk"].T).reshape(-1, heads, dim)
    v = (all_c @ w[p + "uv"].T).reshape(-1, heads, vdim)
    gate = sigmoid(h @ w[p + "g"].T)                              # [T, heads]: one number a head
    out = np.zeros((t, heads, vdim))
    for i in range(t):
        n = start + i + 1                                          # keys 0 .. start + i
        for hd in range(heads):
            s = (k_plain[:n, hd] @ q_plain[i, hd] + all_kr[:n] @ q_rot[i, hd]) * m["scale"]
            top = max(s.max(), w[p + "sink"][hd])
            e = np.exp(s - top)
            out[i, hd] = (e @ v[:n, hd]) / (e.sum() + math.exp(w[p + "sink"][hd] - top))
    out *= gate[:, :, None]
    return out.reshape(t, heads * vdim) @ w[p + "o"].T


# ---------------------------------------------------------------- the windowed attention whose heads talk
def talking_mixer(h, w, p, m, eps, state):
    t = h.shape[0]
    heads, groups, dim, vdim, size = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["mask"]["size"]
    start = state.get("len", 0)
    q = rms_unit(h @ w[p + "q"].T, eps) * w[p + "q.norm"]         # over the whole projection
    k_raw = h @ w[p + "k"].T
    k = rms_unit(k_raw, eps) * w[p + "k.norm"]
    state["k"] = np.concatenate([state["k"], k]) if "k" in state else k
    state["v"] = np.concatenate([state["v"], k_raw]) if "v" in state else k_raw      # the values are the keys before the norm
    state["len"] = start + t
    keys = state["k"].reshape(-1, groups, dim)
    vals = state["v"].reshape(-1, groups, vdim)
    q = q.reshape(t, heads, dim)
    share = heads // groups
    out = np.zeros((t, heads, vdim))
    for i in range(t):
        at = start + i
        lo = max(0, at - size + 1)
        js = np.arange(lo, at + 1)
        weights = np.zeros((heads, len(js)))
        for hd in range(heads):
            s = keys[lo:at + 1, hd // share] @ q[i, hd] * m["scale"]
            s = s - w[p + "r1"][hd] * np.log1p(w[p + "r2"][hd] * (at - js))
            e = np.exp(s - s.max())
            weights[hd] = e / e.sum()
        mixed = w[p + "talk"] @ weights                            # weight_h <- sum_g T[h, g] weight_g
        for hd in range(heads):
            out[i, hd] = mixed[hd] @ vals[lo:at + 1, hd // share]
    out = out.reshape(t, heads * vdim) * sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


# ---------------------------------------------------------------- time mixing with a decay per channel
def time_mixer(h, w, p, m, eps, state):
    t, width = h.shape
    heads, dim = m["heads"], m["dim"]
    prev = state.get("prev", np.zeros(width))
    s_mat = state.get("S", np.zeros((heads, dim, dim)))
    out = np.zeros((t, heads * dim))
    for i in range(t):
        x = h[i]
        mix = {s: x + (prev - x) * w[p + "mu." + s] for s in "rkvgw"}
        r = (w[p + "r"] @ mix["r"]).reshape(heads, dim)
        k = (w[p + "k"] @ mix["k"]).reshape(heads, dim)
        v = (w[p + "v"] @ mix["v"]).reshape(heads, dim)
        gate = silu(w[p + "g"] @ mix["g"])
        decay = np.exp(-np.exp(w[p + "w2"] @ np.tanh(w[p + "w1"] @ mix["w"]) + w[p + "w0"])).reshape(heads, dim)
        o = np.zeros((heads, dim))
        for hd in range(heads):
            kv = np.outer(k[hd], v[hd])
            o[hd] = (s_mat[hd] + w[p + "u"][hd][:, None] * kv).T @ r[hd]
            s_mat[hd] = decay[hd][:, None] * s_mat[hd] + kv
        out[i] = (rms_unit(o, eps).reshape(-1) * w[p + "norm"]) * gate
        prev = x
    state["prev"], state["S"] = prev.copy(), s_mat
    return out @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps, state):
    left = talking_mixer(h, w, p + "left.", m["left"], eps, state.setdefault("left", {}))
    right = time_mixer(h, w, p + "right.", m["right"], eps, state.setdefault("right", {}))
    return m["left_scale"] * left + m["right_scale"] * right


# ---------------------------------------------------------------- the state-space mixer
def mamba2_mixer(h, w, p, m, eps, state):
    t = h.shape[0]
    heads, vdim, n, groups, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = heads * vdim
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * groups * n], proj[:, 2 * inner + 2 * groups * n:]
    tail = state.get("tail", np.zeros((taps - 1, xbc.shape[1])))
    padded = np.concatenate([tail, xbc])
    conv = np.zeros_like(xbc)
    for i in range(t):
        conv[i] = (padded[i:i + taps] * w[p + "conv"].T).sum(0) + w[p + "conv.b"]      # the last column is the current token's
    state["tail"] = padded[len(padded) - (taps - 1):] if taps > 1 else tail
    conv = silu(conv)
    x = conv[:, :inner].reshape(t, heads, vdim)
    b = conv[:, inner:inner + groups * n].reshape(t, groups, n)
    c = conv[:, inner + groups * n:].reshape(t, groups, n)
    dt = softplus(dt + w[p + "dt_bias"])
    s_mat = state.get("S", np.zeros((heads, n, vdim)))
    y = np.zeros((t, heads, vdim))
    per = heads // groups
    for i in range(t):
        for hd in range(heads):
            g = hd // per
            s_mat[hd] = math.exp(-math.exp(w[p + "A_log"][hd]) * dt[i, hd]) * s_mat[hd] + dt[i, hd] * np.outer(b[i, g], x[i, hd])
            y[i, hd] = s_mat[hd].T @ c[i, g] + w[p + "D"][hd] * x[i, hd]
    state["S"] = s_mat
    y = y.reshape(t, inner) * silu(z)                               # the gate comes before the norm
    parts = m["norm_groups"]
    y = rms_unit(y.reshape(t, parts, inner // parts), eps).reshape(t, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


# ---------------------------------------------------------------- feed-forwards
def dense_ff(h, w, p, mlp):
    limit = mlp["limit"]
    g = np.minimum(h @ w[p + "gate"].T + w[p + "gate.b"], limit)
    u = np.clip(h @ w[p + "up"].T + w[p + "up.b"], -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T + w[p + "down.b"]


def route(h, w, p, mlp):
    """The chosen experts and their weights for every token, and every token's gap between the last expert chosen
    and the best left out."""
    top = mlp["router"]["top"]
    z = h @ w[p + "router"].T + w[p + "router.b"]
    order = np.argsort(-z, axis=-1, kind="stable")
    ids = order[:, :top]
    chosen = np.take_along_axis(z, ids, -1)
    e = np.exp(chosen - chosen.max(-1, keepdims=True))
    gap = chosen[:, -1] - np.take_along_axis(z, order[:, top:top + 1], -1)[:, 0] if z.shape[1] > top else np.full(len(z), np.inf)
    return ids, e / e.sum(-1, keepdims=True), gap


def moe_ff(h, w, p, mlp, gaps=None):
    ids, weights, gap = route(h, w, p, mlp)
    if gaps is not None:
        gaps.append(gap)
    out = np.zeros_like(h)
    for i in range(h.shape[0]):
        for e, a in zip(ids[i], weights[i]):
            out[i] += a * (w[f"{p}e{e}.down"] @ gelu_erf(w[f"{p}e{e}.up"] @ h[i]))
    return out


# ---------------------------------------------------------------- the model
MIXERS = {"latent_attention": latent_mixer, "parallel": parallel_mixer, "mamba2": mamba2_mixer}


def forward(cfg, w, tokens, state=None, gaps=None, layers_out=None):
    """Logits [T, vocab] of the next ``tokens`` of one sequence; ``state`` (a dict, empty at the start) carries the
    sequence from call to call.  ``layers_out``: a list that receives the residual after every layer."""
    state = {} if state is None else state
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = w["embed"][np.asarray(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = MIXERS[layer["type"]](x, w, p + "mix.", layer["mixer"], eps, state.setdefault(i, {}))
        x = layer_norm(alpha * x + y, w[p + "norm1"], w[p + "norm1.b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            y = dense_ff(x, w, p + "mlp.", mlp) if mlp["kind"] == "dense" else moe_ff(x, w, p + "mlp.", mlp, gaps)
            x = layer_norm(alpha * x + y, w[p + "norm2"], w[p + "norm2.b"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    logits = x @ w["embed"].T
    cap = cfg.get("logit_softcap")
    return cap * np.tanh(logits / cap) if cap else logits
