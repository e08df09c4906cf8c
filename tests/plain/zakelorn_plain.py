"""Zakelorn written plainly: float64 numpy, one function per mechanism, token by token where a mechanism is
sequential.  It shares nothing with the library: the tests hold the library to it.

``weights`` maps checkpoint names to float64 arrays, ``cfg`` is the dictionary of config.json.
"""
from __future__ import annotations

import math

import numpy as np


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


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


def sees(i, j, size, keep_first):
    """Whether the query at position i sees the key at position j."""
    return j <= i and (i - j < size or j < keep_first)


def sink_attention(q, k, v, positions_q, positions_k, scale, size, keep_first, sinks):
    """q [Tq, H, d], k [Tk, G, d], v [Tk, G, dv]; softmax whose denominator also holds exp(sink_h)."""
    tq, heads, _ = q.shape
    group = heads // k.shape[1]
    seen = np.array([[sees(i, j, size, keep_first) for j in positions_k] for i in positions_q])
    out = np.zeros((tq, heads, v.shape[2]))
    for h in range(heads):
        g = h // group
        s = np.where(seen, (q[:, h] @ k[:, g].T) * scale, -np.inf)
        m = np.maximum(s.max(-1), sinks[h])[:, None]
        e = np.exp(s - m)
        den = e.sum(-1, keepdims=True) + np.exp(sinks[h] - m)
        out[:, h] = (e @ v[:, g]) / den
    return out


def left_mixer(h, positions, w, p, m, eps, past=None):
    """Softmax attention of the tokens ``h`` [T, width] at ``positions`` over themselves and ``past`` = (k, v,
    positions) of the tokens before them.  Returns the result and the new (k, v, positions)."""
    t = h.shape[0]
    heads, kv, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(t, heads, d)
    k = (h @ w[p + "k"].T).reshape(t, kv, d)
    v = (h @ w[p + "v"].T).reshape(t, kv, dv)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}           # no rotation where the mixer names none
    q = rms_unit(rotate_pairs(q, positions, rot["dims"], rot["base"]), eps)
    k = rms_unit(rotate_pairs(k, positions, rot["dims"], rot["base"]), eps)
    if past is not None:
        k, v = np.concatenate([past[0], k]), np.concatenate([past[1], v])
        pos_k = np.concatenate([past[2], positions])
    else:
        pos_k = positions
    mask = m.get("mask") or {}                               # no mask: every earlier token is seen
    size = mask.get("size") if mask.get("size") is not None else math.inf
    o = sink_attention(q, k, v, positions, pos_k, m["scale"], size, mask.get("keep_first", 0), w[p + "sink"])
    o = o.reshape(t, heads * dv) * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T, (k, v, pos_k)


def decayed_state_walk(q, k, v, decay, state):
    """Per head S <- decay_h S + k v^T, o = S^T q, token after token; q, k [T, H, d], v [T, H, dv],
    state [H, d, dv] (changed in place)."""
    t, heads, _ = q.shape
    out = np.zeros((t, heads, v.shape[2]))
    for n in range(t):
        for h in range(heads):
            state[h] = decay[h] * state[h] + np.outer(k[n, h], v[n, h])
            out[n, h] = state[h].T @ q[n, h]
    return out


def right_mixer(h, w, p, m, eps, state):
    t = h.shape[0]
    heads, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).reshape(t, heads, d)
    k = silu(h @ w[p + "k"].T).reshape(t, heads, d)
    v = silu(h @ w[p + "v"].T).reshape(t, heads, dv)
    o = decayed_state_walk(q, k, v, m["decay"], state).reshape(t, heads * dv)
    o = rms_unit(o, eps) * w[p + "norm"] * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def parallel_mixer(h, positions, w, p, m, eps, kept):
    """``kept`` = {"kv": past of the left mixer or None, "state": the right mixer's state}; it is updated."""
    left, kept["kv"] = left_mixer(h, positions, w, p + "left.", m["left"], eps, kept.get("kv"))
    if "state" not in kept:
        r = m["right"]
        kept["state"] = np.zeros((r["heads"], r["dim"], r["vdim"]))
    right = right_mixer(h, w, p + "right.", m["right"], eps, kept["state"])
    return m["left_scale"] * left + m["right_scale"] * right


def dense_ff(h, w, p):
    return gelu_tanh(h @ w[p + "up"].T) @ w[p + "down"].T


def gated_expert(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, w, p, router):
    """For every token the chosen outputs of the router, their weights, and the gap between the worst choice
    score chosen and the best one left out (a close call is one that rounding may turn)."""
    n_out = router["experts"] + router.get("identity", 0)
    z = h @ w[p + "router"].T
    s = np.exp(z - z.max(-1, keepdims=True))
    s = s / s.sum(-1, keepdims=True)
    choice = s + w[p + "correction"]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    per = n_out // groups["count"]
    chosen, weights, gaps = [], [], []
    for t in range(h.shape[0]):
        c = choice[t].copy()
        best = c.reshape(groups["count"], per).max(-1)
        order = sorted(range(groups["count"]), key=lambda g: (-best[g], g))
        gap = math.inf
        if groups["keep"] < groups["count"]:
            gap = best[order[groups["keep"] - 1]] - best[order[groups["keep"]]]
        for g in order[groups["keep"]:]:
            c[g * per:(g + 1) * per] = -math.inf
        ids = sorted(range(n_out), key=lambda e: (-c[e], e))
        top = ids[:router["top"]]
        if router["top"] < n_out and c[ids[router["top"]]] > -math.inf:
            gap = min(gap, c[top[-1]] - c[ids[router["top"]]])
        chosen.append(top)
        weights.append([s[t, e] for e in top])
        gaps.append(gap)
    return chosen, weights, np.array(gaps)


def experts_ff(h, w, p, mlp, gaps_out=None):
    router = mlp["router"]
    chosen, weights, gaps = route(h, w, p, router)
    if gaps_out is not None:
        gaps_out.append(gaps)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(chosen[t], weights[t]):
            if e >= router["experts"]:
                out[t] += wt * h[t]                       # an identity expert
            else:
                out[t] += wt * gated_expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared") is not None:
        out += gated_expert(h, w, p + "shared.") * sigmoid(h @ w[p + "shared.sg"].T)
    return out


def feed_forward(h, w, p, mlp, gaps_out=None):
    if mlp["kind"] == "dense":
        return dense_ff(h, w, p)
    return experts_ff(h, w, p, mlp, gaps_out)


def forward(cfg, w, tokens, kept=None, start=0, layers_out=None, gaps_out=None):
    """Logits [T, vocab] of ``tokens`` that follow ``start`` earlier tokens of the same sequence, whose keys,
    values and states are in ``kept`` (a list with one dictionary per layer, updated in place)."""
    eps = cfg["norm"]["eps"]
    if kept is None:
        kept = [{} for _ in cfg["layers"]]
    positions = np.arange(start, start + len(tokens), dtype=np.float64)
    x = w["embed"][np.asarray(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = parallel_mixer(x, positions, w, p + "mix.", layer["mixer"], eps, kept[i])
        x = x + w[p + "ls1"] * layer_norm(y, w[p + "norm1"], w[p + "norm1.b"], eps)
        if layer.get("mlp") is not None:
            y = feed_forward(x, w, p + "mlp.", layer["mlp"], gaps_out)
            x = x + w[p + "ls2"] * layer_norm(y, w[p + "norm2"], w[p + "norm2.b"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return x @ w["embed"].T


def token_by_token(cfg, w, tokens):
    kept = [{} for _ in cfg["layers"]]
    return np.concatenate([forward(cfg, w, tokens[n:n + 1], kept, n) for n in range(len(tokens))])
