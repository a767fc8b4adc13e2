"""Small Bosalix configurations with sizes and constants of their own, and random weights for them."""
from __future__ import annotations

import json
import os

import numpy as np
import torch


def stretch(factor=4.0, original=64, low=1.0, high=4.0):
    return {"factor": factor, "original": original, "low": low, "high": high}


def attention(heads, kv_heads, dim, vdim, scale=None, rot=None, base=10000.0, scaling=None, window=None, keep_first=None,
              v_mix=False):
    r = {"dims": dim if rot is None else rot, "base": base}
    if scaling is not None:
        r["scaling"] = scaling
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale, "rot": r}
    if window is not None:
        m["mask"] = {"size": window}
        if keep_first is not None:
            m["mask"]["keep_first"] = keep_first
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m}


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale=None, base=10000.0, window=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": (dim + rot_dim) ** -0.5 if scale is None else scale, "rot": {"dims": rot_dim, "base": base}}
    if window is not None:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m}


def moe(experts, top, ff, identity=None):
    router = {"experts": experts, "top": top}
    if identity is not None:
        router["identity"] = identity
    return {"kind": "moe", "router": router, "expert": {"ff": ff}}


def config(width, vocab, layers, eps=1e-5, embedding_scale=1.0, residual_mult=1.0):
    """``layers``: (mixer entry, mlp or None)."""
    return {"architecture": "Bosalix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": residual_mult,
            "embedding": {"scale": embedding_scale}, "layers": [{**mixer, "mlp": mlp} for mixer, mlp in layers]}


CASES = {
    # each mechanism by itself
    "latent_only": config(64, 96, [(latent(4, 16, 8, 16, 24, 20, window=40), None)], residual_mult=0.7),
    "attention_only": config(64, 96, [(attention(4, 2, 16, 16, rot=8, window=33, keep_first=5, scaling=stretch()), None)],
                             embedding_scale=3.0),
    "experts_behind_attention": config(48, 60, [(attention(2, 1, 8, 24, window=20, keep_first=1), moe(5, 3, 20, identity=3))],
                                       residual_mult=0.25),
    # values mixed over three layers, a latent layer between them; unequal key widths among the mixing layers
    "mixed_values": config(64, 80, [(attention(4, 2, 16, 8, v_mix=True, window=70, keep_first=3), moe(4, 2, 24, identity=1)),
                                    (latent(2, 8, 4, 12, 10, 12), None),
                                    (attention(2, 2, 32, 8, rot=16, v_mix=True, scaling=stretch(8.0, 32, 1.0, 2.0)), moe(3, 1, 16)),
                                    (attention(4, 2, 16, 8, rot=4, v_mix=True, window=64, keep_first=64), None)],
                           embedding_scale=2.0, residual_mult=0.5),
    # no window anywhere, one head, all experts chosen, no identity experts, attention without v_mix behind one with it
    "plain_sizes": config(40, 50, [(attention(1, 1, 8, 8, v_mix=True), moe(2, 2, 12, identity=0)),
                                   (attention(3, 3, 16, 16, rot=0), moe(6, 2, 8, identity=2)),
                                   (latent(1, 16, 2, 8, 12, 8, window=1), moe(1, 1, 24, identity=4))], eps=1e-6),
    # wide heads, windows at a page's border and beyond it, the kept positions beyond a page
    "wide": config(192, 300, [(latent(4, 64, 32, 64, 112, 72, window=65), moe(8, 4, 64, identity=4)),
                              (attention(6, 2, 64, 48, rot=32, window=64, keep_first=70, v_mix=True, scaling=stretch(8.0, 256)), None),
                              (attention(6, 2, 128, 48, rot=64, window=130, keep_first=6, v_mix=True, base=500.0), moe(4, 2, 96)),
                              (latent(2, 128, 64, 128, 200, 100), None)],
                   embedding_scale=8.0, residual_mult=0.5),
}


def tensor_shapes(cfg: dict) -> dict[str, tuple[int, ...]]:
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "head": (V, W), "final.norm": (W,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (W,)
        out[p + "shift"] = (W,)
        H, K, Vd = m["heads"], m["dim"], m["vdim"]
        if layer["type"] == "latent_attention":
            R, rank, qr = m["rot_dim"], m["kv_rank"], m["q_rank"]
            out.update({p + "mix.dq": (qr, W), p + "mix.dq.norm": (qr,), p + "mix.uq": (H * (K + R), qr),
                        p + "mix.dkv": (rank + R, W), p + "mix.dkv.norm": (rank,), p + "mix.uk": (H * K, rank),
                        p + "mix.uv": (H * Vd, rank), p + "mix.o": (W, H * Vd)})
        else:
            G = m["kv_heads"]
            out.update({p + "mix.q": (H * K, W), p + "mix.q.b": (H * K,), p + "mix.k": (G * K, W), p + "mix.k.b": (G * K,),
                        p + "mix.v": (G * Vd, W), p + "mix.v.b": (G * Vd,), p + "mix.q.norm": (K,), p + "mix.k.norm": (K,),
                        p + "mix.pb": (H,), p + "mix.o": (W, H * Vd), p + "mix.o.b": (W,)})
            if m.get("v_mix"):
                out[p + "mix.vmix"] = ()
        f = layer.get("mlp")
        if f is not None:
            out[p + "norm2"] = (W,)
            E, I = f["router"]["experts"], f["router"].get("identity", 0)
            out[p + "mlp.router"] = (E + I, W)
            out[p + "mlp.correction"] = (E + I,)
            for e in range(E):
                out[f"{p}mlp.e{e}.up"] = (f["expert"]["ff"], W)
                out[f"{p}mlp.e{e}.down"] = (W, f["expert"]["ff"])
    return out


def random_weights(cfg: dict, seed: int, dtype=torch.float32) -> dict[str, torch.Tensor]:
    """Weights that keep every mechanism alive: products of unit scale, norm weights around zero, shifts between 0 and 1,
    score biases that leave the sigmoid weights small, mixes between 0 and 1, corrections of the size of the scores."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if last in ("norm1", "norm2") or name == "final.norm":
            a = 0.3 * rng.standard_normal(shape)
        elif name.endswith(".norm"):            # the latents' and the heads' norms: plain weights
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif last == "shift":
            a = rng.uniform(0.0, 1.0, shape)
        elif last == "pb":
            a = -2.0 + rng.standard_normal(shape)
        elif last == "vmix":
            a = rng.uniform(0.2, 0.8, shape)
        elif last == "correction":
            a = 0.2 * rng.standard_normal(shape)
        elif last == "b":
            a = 0.3 * rng.standard_normal(shape)
        elif name == "embed":
            a = rng.standard_normal(shape)
        elif last == "router":
            a = 2.0 * rng.standard_normal(shape) / np.sqrt(shape[-1])
        else:
            a = rng.standard_normal(shape) / np.sqrt(shape[-1])
        out[name] = torch.from_numpy(np.asarray(a, dtype=np.float64)).to(torch.bfloat16).to(dtype)      # bfloat16 numbers, whatever the type
    return out


def tokens(cfg: dict, n: int, seed: int) -> list[int]:
    """Token ids from 2 on (0 and 1 are kept for the tests that plant a token)."""
    rng = np.random.default_rng(1000 + seed)
    return [int(t) for t in rng.integers(2, cfg["vocab"], size=n)]


def random_case(seed: int) -> dict:
    """A configuration drawn at random: two to four layers of either kind with sizes of many kinds."""
    rng = np.random.default_rng(seed)
    pick = lambda *xs: xs[int(rng.integers(len(xs)))]
    width = pick(24, 40, 64, 72, 128)
    layers, mixing = [], None
    for _ in range(int(rng.integers(2, 5))):
        f = pick(None, moe(pick(1, 3, 4, 8), 1, pick(8, 20, 32), identity=pick(None, 0, 1, 3)))
        if f is not None:
            f["router"]["top"] = int(rng.integers(1, f["router"]["experts"] + f["router"].get("identity", 0) + 1))
        if rng.random() < 0.5:
            rot = pick(2, 4, 8, 16)
            layers.append((latent(pick(1, 2, 3, 4), pick(4, 8, 16, 24), rot, pick(4, 8, 16, 20), pick(6, 16, 24, 40), pick(5, 8, 16, 24),
                                  scale=pick(0.1, 0.25, 1.0), base=pick(100.0, 10000.0), window=pick(None, 1, 7, 64, 65, 100)), f))
        else:
            kv = pick(1, 2)
            dim = pick(4, 8, 16, 32, 48)
            mix = bool(rng.random() < 0.6)
            vdim = pick(4, 8, 16, 24) if not mix or mixing is None else mixing[1]
            kv = kv if not mix or mixing is None else mixing[0]
            if mix and mixing is None:
                mixing = (kv, vdim)
            window = pick(None, 2, 9, 64, 65, 90)
            layers.append((attention(kv * pick(1, 2, 3), kv, dim, vdim, scale=pick(0.1, 0.3, 1.0), rot=pick(0, 2, dim // 2, dim),
                                     base=pick(50.0, 10000.0), scaling=pick(None, stretch(pick(2.0, 8.0), pick(16, 64), 1.0, pick(2.0, 4.0))),
                                     window=window, keep_first=pick(None, 0, 1, 4, 70), v_mix=mix), f))
    return config(width, int(rng.integers(30, 200)), layers, eps=pick(1e-6, 1e-5), embedding_scale=pick(1.0, 4.0, 0.5),
                  residual_mult=pick(1.0, 0.5, 0.3))


def write_model_dir(path: str, cfg: dict, weights: dict[str, torch.Tensor]) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f)
    save_file({n: t.contiguous() for n, t in weights.items()}, os.path.join(path, "model.safetensors"))
    return path


def as_float64(weights: dict[str, torch.Tensor]) -> dict[str, np.ndarray]:
    return {n: t.to(torch.float64).numpy() for n, t in weights.items()}
