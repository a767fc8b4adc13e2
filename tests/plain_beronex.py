"""A plain, slow implementation of the Beronex design: float64, whole sequences, no cache, one function per mechanism.

It is written from the design's formulas and shares nothing with the library; the library's logits are held against it.
``w`` maps tensor names to float64 arrays; a linear weight is [out, in] and applied as ``W x``.

embedding:    x = embed[token] * embedding.scale
A layer:      x <- x + norm1b(mixer(norm1(x)));  x <- x + norm2b(ff(norm2(x)))      (the second half optional)
norm:         y / sqrt(mean(y^2) + eps) * weight
rotation:     frequencies f_i = base^(-2i / dims), bent by YaRN (below); a pair (u, v) at position p becomes
              (u cos a - v sin a, v cos a + u sin a) * m with a = p f_i and m = 0.1 ln(factor) + 1
lightning:    q, k, v = silu(W h);  per head S <- decay_h S + k v^T, o = S^T q;  all heads normed together with a weight,
              times sigmoid(W_g h);  W_o
latent:       c_q = norm(W_dq h), q = W_uq c_q, per head [dim plain | rot_dim rotated in halves];  W_dkv h gives the latent
              c = norm(first kv_rank) and one rotated key part (the rest, no norm) for all heads;  k_h = [W_uk,h c | that
              part], v_h = W_uv,h c;  score = q . k * scale, j <= i;  softmax;  W_o
attention:    q, k, v = W h;  the first rot.dims dimensions of a head rotated in neighbouring pairs;  q and k divided by
              their root mean square over the head;  score = q . k * scale for 0 <= i - j < mask.size;  softmax;  head h
              times sigmoid(W_g h)_h;  W_o.  ``kv_from``: the keys and values are another layer's.
dense ff:     W_down (gelu_tanh(W_gate h) * (W_up h))
experts:      z = W_router h + b;  the ``top`` largest, weights softmax over them;  expert: g = min(W_gate h, limit),
              u = clamp(W_up h, -limit, limit), W_down (g sigmoid(1.702 g) (u + 1))
logits:       head . norm(x)
"""
from __future__ import annotations

import math

import numpy as np


def rms_norm(y: np.ndarray, weight, eps: float) -> np.ndarray:
    out = y / np.sqrt(np.mean(y * y, axis=-1, keepdims=True) + eps)
    return out if weight is None else out * weight


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotation_table(rot: dict) -> tuple[np.ndarray, float]:
    """The frequency of every pair and the factor on cosine and sine."""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    s = rot.get("scaling")
    if s is None:
        return f, 1.0

    def where(turns):      # the (fractional) pair that makes this many turns over the original length
        return dims * math.log(s["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(where(s["fast"])), 0)
    hi = min(math.ceil(where(s["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / s["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(s["factor"]) + 1.0


def rotate(x: np.ndarray, positions: np.ndarray, rot: dict, layout: str) -> np.ndarray:
    """x [T, heads, n]: the first rot.dims numbers of every head turned, pair i being (2i, 2i+1) ("pairs") or
    (i, i + dims/2) ("halves")."""
    dims = rot["dims"]
    f, m = rotation_table(rot)
    out = x.copy()
    for i in range(dims // 2):
        a, b = (2 * i, 2 * i + 1) if layout == "pairs" else (i, i + dims // 2)
        ang = positions * f[i]
        c, s = (np.cos(ang) * m)[:, None], (np.sin(ang) * m)[:, None]
        out[:, :, a] = x[:, :, a] * c - x[:, :, b] * s
        out[:, :, b] = x[:, :, b] * c + x[:, :, a] * s
    return out


def masked_softmax(scores: np.ndarray, window: int | None) -> np.ndarray:
    """scores [T, T]: row i sees columns j <= i, and with a window only those with i - j < window."""
    T = scores.shape[0]
    out = np.zeros_like(scores)
    for i in range(T):
        lo = 0 if window is None else max(0, i - window + 1)
        row = scores[i, lo:i + 1]
        e = np.exp(row - row.max())
        out[i, lo:i + 1] = e / e.sum()
    return out


def lightning(h: np.ndarray, m: dict, w: dict, p: str, eps: float, state=None, return_state: bool = False):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).reshape(T, H, D)
    k = silu(h @ w[p + "k"].T).reshape(T, H, D)
    v = silu(h @ w[p + "v"].T).reshape(T, H, V)
    o = np.zeros((T, H, V))
    states = np.zeros((H, D, V))
    for head in range(H):
        S = np.zeros((D, V)) if state is None else state[head].copy()
        for t in range(T):
            S = m["decay"][head] * S + np.outer(k[t, head], v[t, head])
            o[t, head] = S.T @ q[t, head]
        states[head] = S
    o = rms_norm(o.reshape(T, H * V), w[p + "norm"], eps) * sigmoid(h @ w[p + "g"].T)
    out = o @ w[p + "o"].T
    return (out, states) if return_state else out


def latent_attention(h: np.ndarray, m: dict, w: dict, p: str, eps: float) -> np.ndarray:
    T = h.shape[0]
    H, D, R, V, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = np.arange(T, dtype=np.float64)
    q = (rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps) @ w[p + "uq"].T).reshape(T, H, D + R)
    down = h @ w[p + "dkv"].T
    c = rms_norm(down[:, :C], w[p + "dkv.norm"], eps)
    k_rot = rotate(down[:, None, C:], pos, m["rot"], "halves")[:, 0]           # [T, R], one for all heads
    q_rot = rotate(q[:, :, D:], pos, m["rot"], "halves")
    k = (c @ w[p + "uk"].T).reshape(T, H, D)
    v = (c @ w[p + "uv"].T).reshape(T, H, V)
    out = np.zeros((T, H, V))
    for head in range(H):
        scores = (q[:, head, :D] @ k[:, head].T + q_rot[:, head] @ k_rot.T) * m["scale"]
        out[:, head] = masked_softmax(scores, None) @ v[:, head]
    return out.reshape(T, H * V) @ w[p + "o"].T


def attention_keys_values(h: np.ndarray, m: dict, w: dict, p: str, eps: float):
    """Keys as a cache would hold them (rotated, then divided by their root mean square) and values."""
    T = h.shape[0]
    G, D, V = m["kv_heads"], m["dim"], m["vdim"]
    k = rotate((h @ w[p + "k"].T).reshape(T, G, D), np.arange(T, dtype=np.float64), m["rot"], "pairs")
    return rms_norm(k, None, eps), (h @ w[p + "v"].T).reshape(T, G, V)


def attention(h: np.ndarray, keys: np.ndarray, values: np.ndarray, m: dict, w: dict, p: str, eps: float) -> np.ndarray:
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rotate((h @ w[p + "q"].T).reshape(T, H, D), np.arange(T, dtype=np.float64), m["rot"], "pairs")
    q = rms_norm(q, None, eps)
    gate = sigmoid(h @ w[p + "g"].T)                                            # [T, H]
    window = m["mask"]["size"] if m.get("mask") is not None else None
    out = np.zeros((T, H, V))
    for head in range(H):
        g = head // (H // G)
        out[:, head] = masked_softmax(q[:, head] @ keys[:, g].T * m["scale"], window) @ values[:, g]
    return (out * gate[:, :, None]).reshape(T, H * V) @ w[p + "o"].T


def dense_ff(h: np.ndarray, w: dict, p: str) -> np.ndarray:
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h: np.ndarray, f: dict, w: dict, p: str):
    """The chosen experts [T, top] (best first) and their weights."""
    z = h @ w[p + "router"].T + w[p + "router.b"]
    top = f["router"]["top"]
    ids = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    chosen = np.take_along_axis(z, ids, axis=-1)
    e = np.exp(chosen - chosen.max(axis=-1, keepdims=True))
    return ids, e / e.sum(axis=-1, keepdims=True), z


def expert(h: np.ndarray, w: dict, p: str, limit: float) -> np.ndarray:
    g = np.minimum(h @ w[p + "gate"].T, limit)
    u = np.clip(h @ w[p + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def experts_ff(h: np.ndarray, f: dict, w: dict, p: str) -> np.ndarray:
    ids, weights, _ = route(h, f, w, p)
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, wt in zip(ids[t], weights[t]):
            out[t] += wt * expert(h[t:t + 1], w, f"{p}e{e}.", f["expert"]["limit"])[0]
    return out


def forward(cfg: dict, w: dict, tokens, return_layers: bool = False):
    """Logits [T, vocab] of a whole sequence (and the residual stream behind every layer)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    kept, streams = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        h = rms_norm(x, w[f"l{i}.norm1"], eps)
        if layer["type"] == "lightning":
            y = lightning(h, m, w, p, eps)
        elif layer["type"] == "latent_attention":
            y = latent_attention(h, m, w, p, eps)
        elif layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = attention_keys_values(h, m, w, p, eps)
            y = attention(h, *kept[i if src is None else src], m, w, p, eps)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, w[f"l{i}.norm1b"], eps)
        f = layer.get("mlp")
        if f is not None:
            h = rms_norm(x, w[f"l{i}.norm2"], eps)
            y = dense_ff(h, w, f"l{i}.mlp.") if f["kind"] == "dense" else experts_ff(h, f, w, f"l{i}.mlp.")
            x = x + rms_norm(y, w[f"l{i}.norm2b"], eps)
        streams.append(x.copy())
    logits = rms_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, streams) if return_layers else logits
