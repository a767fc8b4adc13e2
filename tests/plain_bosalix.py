"""A plain, slow implementation of the Bosalix design: float64, whole sequences, no cache, one function per mechanism.

It is written from the design's formulas and shares nothing with the library; the library's logits are held against it.
``w`` maps tensor names to float64 arrays; a linear weight is [out, in] and applied as ``W x``.

embedding:    x = embed[token] * embedding.scale
a layer:      x <- x + m unit(mixer(shift(x))) (1 + norm1);  x <- x + m unit(ff(x)) (1 + norm2)   (m = residual_mult;
              unit(y) = y / sqrt(mean(y^2) + eps); the second half optional)
shift:        h_t <- h_t + (h_(t-1) - h_t) * shift, h_(-1) = 0, the h on the right being the rows before the shift
latent:       c_q = unit(W_dq h) dq.norm, q = W_uq c_q, per head [dim plain | rot_dim rotated in neighbouring pairs];
              W_dkv h gives the latent c = unit(first kv_rank) dkv.norm and one rotated key part (the rest, no norm) for all
              heads;  k_h = [W_uk,h c | that part], v_h = W_uv,h c;  score = q . k * scale for 0 <= i - j < mask.size;
              softmax;  W_o
attention:    q, k, v = W h + b;  q and k normed per head with one weight for all heads;  the first rot.dims dimensions
              of a head rotated, i paired with i + dims/2, frequencies stretched as in Llama 3.1;  every value head divided
              by its root mean square;  v <- (1 - vmix) v + vmix v_first in every v_mix layer but the first of them;
              weight of key j for query i: sigmoid(q . k * scale + pb_h) if j <= i and (i - j < mask.size or
              j < mask.keep_first), not normalised;  W_o + b
experts:      s = softmax(W_router h) over experts and identity experts;  the ``top`` largest s + correction are chosen;
              out = sum of s_e expert_e(h) over the chosen, expert_e(h) = W_down gelu(W_up h) (erf form) or h itself for
              the identity experts, which are the last ones
logits:       head . (unit(x) (1 + final.norm))
"""
from __future__ import annotations

import math

import numpy as np


def unit(y: np.ndarray, eps: float) -> np.ndarray:
    return y / np.sqrt(np.mean(y * y, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


_erf = np.vectorize(math.erf, otypes=[np.float64])


def gelu(z):
    return 0.5 * z * (1.0 + _erf(z / math.sqrt(2.0)))


def frequencies(rot: dict) -> np.ndarray:
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    s = rot.get("scaling")
    if s is None:
        return f
    out = f.copy()
    for i, fi in enumerate(f):
        length = 2.0 * math.pi / fi
        if length < s["original"] / s["high"]:
            continue
        if length > s["original"] / s["low"]:
            out[i] = fi / s["factor"]
        else:
            t = (s["original"] / length - s["low"]) / (s["high"] - s["low"])
            out[i] = (1.0 - t) * fi / s["factor"] + t * fi
    return out


def rotate(x: np.ndarray, positions: np.ndarray, rot: dict, layout: str) -> np.ndarray:
    """x [T, heads, n]: the first rot.dims numbers of every head turned, pair i being (2i, 2i+1) ("pairs") or
    (i, i + dims/2) ("halves")."""
    dims = rot["dims"]
    f = frequencies(rot)
    out = x.copy()
    for i in range(dims // 2):
        a, b = (2 * i, 2 * i + 1) if layout == "pairs" else (i, i + dims // 2)
        ang = positions * f[i]
        c, s = np.cos(ang)[:, None], np.sin(ang)[:, None]
        out[:, :, a] = x[:, :, a] * c - x[:, :, b] * s
        out[:, :, b] = x[:, :, b] * c + x[:, :, a] * s
    return out


def visible(T: int, window: int | None, keep_first: int = 0) -> np.ndarray:
    """[T, T] of booleans: whether query i sees key j."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    near = (i - j < window) if window is not None else np.ones((T, T), dtype=bool)
    return (j <= i) & (near | (j < keep_first))


def token_shift(h: np.ndarray, shift: np.ndarray) -> np.ndarray:
    before = np.concatenate([np.zeros_like(h[:1]), h[:-1]])
    return h + (before - h) * shift


def latent_attention(h, m: dict, w: dict, p: str, eps: float):
    T = h.shape[0]
    H, K, R, V, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = np.arange(T, dtype=np.float64)
    cq = unit(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).reshape(T, H, K + R)
    down = h @ w[p + "dkv"].T
    c = unit(down[:, :rank], eps) * w[p + "dkv.norm"]
    k_rot = down[:, rank:].reshape(T, 1, R)
    if R:
        q = np.concatenate([q[:, :, :K], rotate(q[:, :, K:], pos, m["rot"], "pairs")], axis=2)
        k_rot = rotate(k_rot, pos, m["rot"], "pairs")
    k = (c @ w[p + "uk"].T).reshape(T, H, K)
    v = (c @ w[p + "uv"].T).reshape(T, H, V)
    see = visible(T, (m.get("mask") or {}).get("size"))
    out = np.zeros((T, H, V))
    for hh in range(H):
        s = (q[:, hh, :K] @ k[:, hh].T + q[:, hh, K:] @ k_rot[:, 0].T) * m["scale"]
        s = np.where(see, s, -np.inf)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, hh] = (e / e.sum(axis=1, keepdims=True)) @ v[:, hh]
    return out.reshape(T, H * V) @ w[p + "o"].T


def attention(h, m: dict, w: dict, p: str, eps: float, v_first):
    """Returns the mixer's output and the values it kept (what a later v_mix layer mixes in if this is the first)."""
    T = h.shape[0]
    H, G, K, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = np.arange(T, dtype=np.float64)
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, K)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, K)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, V)
    q = unit(q, eps) * w[p + "q.norm"]
    k = unit(k, eps) * w[p + "k.norm"]
    rot = m.get("rot")
    if rot is not None and rot["dims"] > 0:
        q, k = rotate(q, pos, rot, "halves"), rotate(k, pos, rot, "halves")
    v = unit(v, eps)
    if m.get("v_mix") and v_first is not None:
        lam = float(w[p + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    mask = m.get("mask") or {}
    see = visible(T, mask.get("size"), mask.get("keep_first", 0))
    out = np.zeros((T, H, V))
    for hh in range(H):
        g = hh // (H // G)
        s = q[:, hh] @ k[:, g].T * m["scale"] + w[p + "pb"][hh]
        out[:, hh] = np.where(see, sigmoid(s), 0.0) @ v[:, g]
    return out.reshape(T, H * V) @ w[p + "o"].T + w[p + "o.b"], v


def experts(h, f: dict, w: dict, p: str):
    E, I, top = f["router"]["experts"], f["router"].get("identity", 0), f["router"]["top"]
    z = h @ w[p + "router"].T
    e = np.exp(z - z.max(axis=1, keepdims=True))
    s = e / e.sum(axis=1, keepdims=True)
    choice = s + w[p + "correction"]
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for x in np.argsort(-choice[t], kind="stable")[:top]:
            if x >= E:
                out[t] += s[t, x] * h[t]
            else:
                out[t] += s[t, x] * (w[f"{p}e{x}.down"] @ gelu(w[f"{p}e{x}.up"] @ h[t]))
    return out


def forward(cfg: dict, w: dict, tokens, layers_out: list | None = None) -> np.ndarray:
    """Logits [T, vocab] of one sequence; ``layers_out`` collects the stream behind every layer."""
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = w["embed"][np.asarray(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = token_shift(x, w[p + "shift"])
        if layer["type"] == "latent_attention":
            y = latent_attention(h, layer["mixer"], w, p + "mix.", eps)
        else:
            y, v = attention(h, layer["mixer"], w, p + "mix.", eps, v_first)
            if layer["mixer"].get("v_mix") and v_first is None:
                v_first = v
        x = x + mult * unit(y, eps) * (1.0 + w[p + "norm1"])
        if layer.get("mlp") is not None:
            x = x + mult * unit(experts(x, layer["mlp"], w, p + "mlp."), eps) * (1.0 + w[p + "norm2"])
        if layers_out is not None:
            layers_out.append(x.copy())
    return (unit(x, eps) * (1.0 + w["final.norm"])) @ w["head"].T
