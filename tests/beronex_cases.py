"""Small Beronex configurations with sizes and constants of their own, and random weights for them."""
from __future__ import annotations

import json
import os

import numpy as np
import torch


def yarn(factor=4.0, original=64, fast=16.0, slow=1.0):
    return {"factor": factor, "original": original, "fast": fast, "slow": slow}


def attention(heads, kv_heads, dim, vdim, scale=None, rot=None, base=10000.0, scaling=None, window=None, kv_from=None):
    r = {"dims": dim if rot is None else rot, "base": base}
    if scaling is not None:
        r["scaling"] = scaling
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale, "rot": r}
    if window is not None:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale=None, base=10000.0, scaling=None):
    r = {"dims": rot_dim, "base": base}
    if scaling is not None:
        r["scaling"] = scaling
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                      "scale": (dim + rot_dim) ** -0.5 if scale is None else scale, "rot": r}}


def lightning(heads, dim, vdim, decay):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit=2.0):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}


def config(width, vocab, layers, eps=1e-5, embedding_scale=1.0):
    """``layers``: (mixer entry, mlp or None)."""
    return {"architecture": "Beronex", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": embedding_scale}, "layers": [{**mixer, "mlp": mlp} for mixer, mlp in layers]}


CASES = {
    # each mechanism by itself
    "lightning_only": config(64, 96, [(lightning(4, 16, 16, [0.5, 0.9, 0.99, 1.0]), None)], embedding_scale=3.0),
    "latent_only": config(64, 96, [(latent(4, 16, 8, 16, 24, 20, scaling=yarn()), None)]),
    "attention_only": config(64, 96, [(attention(4, 2, 16, 16, rot=8, window=40, scaling=yarn(8.0, 32, 8.0, 2.0)), None)]),
    "dense_behind_attention": config(40, 50, [(attention(1, 1, 8, 8), dense(24))], embedding_scale=0.5),
    "experts_behind_lightning": config(48, 60, [(lightning(2, 8, 24, [0.8, 0.97]), moe(6, 2, 20, limit=0.7))]),
    # sizes that are no multiples of 16, 8 or 4; value width other than key width; one kv head and as many as heads; a
    # whole head rotated, a part, with and without stretched frequencies; windows below and above a page, and none; layers
    # on another layer's keys with a narrower, an equal and a wider window; a latent and a query latent that are no
    # multiples of 8; decays of 0 and 1; one expert, all experts chosen; layers without a feed-forward
    "odd": config(72, 101, [
        (lightning(3, 20, 12, [0.0, 0.95, 1.0]), dense(36)),
        (latent(3, 12, 4, 20, 40, 13, scale=0.4, base=500.0), None),
        (attention(6, 3, 20, 28, rot=12, base=500.0, scale=0.31, window=70), moe(5, 5, 18, limit=1.5)),
        (attention(6, 3, 20, 28, rot=12, base=500.0, scale=0.5, window=9, kv_from=2), dense(30)),
        (latent(2, 24, 6, 12, 18, 9, scaling=yarn(2.0, 16, 4.0, 1.0)), moe(1, 1, 10, limit=3.0)),
        (attention(6, 3, 20, 28, rot=12, base=500.0, window=100, kv_from=2), None),
        (attention(3, 3, 24, 8, rot=24, scaling=yarn(16.0, 40, 10.0, 0.5)), None),
        (attention(3, 3, 24, 8, rot=24, scaling=yarn(16.0, 40, 10.0, 0.5), window=33, kv_from=6), moe(7, 3, 12)),
    ], embedding_scale=4.0),
    # a width that is no multiple of four, heads of 10, windows of one token and of a page
    "ragged": config(50, 67, [
        (attention(5, 5, 10, 10, rot=10, base=77.0, window=64), dense(10)),
        (lightning(2, 40, 24, [0.999, 0.6]), moe(4, 3, 14, limit=0.5)),
        (lightning(3, 8, 70, [0.3, 0.9, 0.99]), None),
        (latent(5, 10, 2, 6, 50, 30), dense(22)),
        (attention(2, 1, 6, 14, rot=2, window=1), None),
        (attention(5, 5, 10, 10, rot=10, base=77.0, window=65, kv_from=0), None),
    ], eps=1e-6, embedding_scale=7.0),
    # heads as wide as served models have them
    "wide": config(256, 300, [
        (lightning(2, 128, 128, [0.97, 0.999]), dense(512)),
        (attention(4, 1, 128, 128, rot=64, base=1e6, window=200, scaling=yarn(8.0, 128, 32.0, 1.0)), None),
        (latent(4, 128, 64, 128, 256, 96, scaling=yarn(40.0, 100, 32.0, 1.0)), moe(8, 2, 128)),
        (lightning(1, 256, 40, [0.99]), None),
        (attention(4, 1, 128, 128, rot=64, base=1e6, window=300, scaling=yarn(8.0, 128, 32.0, 1.0), kv_from=1), dense(256)),
        (latent(2, 32, 16, 48, 304, 200), None),
    ], embedding_scale=10.0),
    # as a served model's layers might be laid out, small
    "regular": config(128, 256, [
        (latent(4, 32, 16, 32, 48, 40, scaling=yarn(8.0, 128, 32.0, 1.0), base=1e5), dense(192)),
        (lightning(4, 32, 48, [0.8, 0.9, 0.99, 0.999]), moe(8, 2, 64)),
        (attention(4, 2, 32, 32, window=80, scaling=yarn(4.0, 64, 16.0, 1.0)), dense(192)),
        (latent(4, 32, 16, 32, 48, 40, base=1e5), moe(8, 3, 64, limit=1.0)),
        (attention(4, 2, 32, 32, window=80, scaling=yarn(4.0, 64, 16.0, 1.0), kv_from=2), dense(320)),
    ], embedding_scale=9.0),
}


def random_case(seed: int) -> dict:
    """A configuration drawn from sizes of many kinds."""
    rng = np.random.default_rng(7000 + seed)
    pick = lambda xs: xs[int(rng.integers(len(xs)))]
    divisors = lambda n: [d for d in range(1, n + 1) if n % d == 0]
    width = pick([40, 56, 64, 90, 96, 120, 160, 200, 256])
    layers = []
    for i in range(int(rng.integers(2, 7))):
        r = rng.random()
        mlp = None if r < 0.2 else dense(pick([8, 20, 24, 40, 64, 100, 130])) if r < 0.6 else \
            (lambda e: moe(e, int(rng.integers(1, e + 1)), pick([8, 12, 24, 40, 72]), limit=pick([0.5, 1.0, 2.0, 7.0])))(pick([1, 2, 3, 4, 8, 11, 16]))
        heads = pick([1, 2, 3, 4, 6, 8])
        scaling = None if rng.random() < 0.3 else yarn(pick([2.0, 4.0, 8.0, 32.0]), pick([16, 64, 512, 4096]), pick([8.0, 32.0]), pick([0.5, 1.0, 2.0]))
        base = pick([100.0, 1e4, 5e5])
        kind = rng.random()
        own = [j for j, (l, _) in enumerate(layers) if l["type"] == "attention" and "kv_from" not in l["mixer"]]
        if kind < 0.25:
            layers.append((lightning(heads, pick([4, 8, 16, 20, 32, 48, 64]), pick([4, 8, 16, 24, 32, 64, 96]),
                                     [float(rng.choice([0.5, 0.9, 0.99, 0.999, 1.0])) for _ in range(heads)]), mlp))
        elif kind < 0.5:
            dim = pick([4, 8, 16, 24, 32, 64])
            layers.append((latent(heads, dim, pick([2, 4, 8, 16, 32]), pick([4, 8, 16, 24, 32, 64]), pick([8, 16, 20, 48, 64, 100, 128]),
                                  pick([5, 8, 24, 33, 64, 80]), scale=float(rng.uniform(0.5, 1.5)) * dim ** -0.5, base=base,
                                  scaling=scaling), mlp))
        elif own and rng.random() < 0.5:
            src = layers[pick(own)]
            m = src[0]["mixer"]
            layers.append((attention(m["heads"], m["kv_heads"], m["dim"], m["vdim"], scale=float(rng.uniform(0.5, 1.5)) * m["dim"] ** -0.5,
                                     rot=m["rot"]["dims"], base=m["rot"]["base"], scaling=m["rot"].get("scaling"),
                                     window=pick([None, 3, 17, 64, 72, 130]), kv_from=layers.index(src)), mlp))
        else:
            dim = pick([4, 8, 12, 16, 24, 32, 40, 48, 64, 80, 96])
            layers.append((attention(heads, pick(divisors(heads)), dim, pick([4, 8, 16, 24, 32, 48, 64, 72, 96]),
                                     scale=float(rng.uniform(0.5, 1.5)) * dim ** -0.5, rot=pick([2, max(2, dim // 2 // 2 * 2), dim]),
                                     base=base, scaling=scaling, window=pick([None, 2, 31, 64, 65, 100, 128])), mlp))
    return config(width, int(rng.integers(50, 500)), layers, eps=pick([1e-5, 1e-6]), embedding_scale=pick([1.0, 3.0, 12.0]))


def tensors(cfg: dict, seed: int, peaky: float = 1.0) -> dict[str, np.ndarray]:
    """Random weights as float64 arrays whose values are bfloat16 numbers.  ``peaky`` scales the latent attentions' queries, so that
    single keys decide a row of the softmax (the other attention norms its queries: there the scale does it)."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    out = {}

    def put(name, shape, std=1.0, mean=0.0):
        v = torch.tensor(rng.normal(mean, std, size=shape), dtype=torch.float32).to(torch.bfloat16)
        out[name] = v.to(torch.float64).numpy()

    put("embed", (cfg["vocab"], W))
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        for n in ("norm1", "norm1b"):
            put(p + n, (W,), 0.1, 1.0)
        H, D, V = m["heads"], m["dim"], m["vdim"]
        if layer["type"] == "attention":
            G = m["kv_heads"]
            put(p + "mix.q", (H * D, W), W ** -0.5)
            if m.get("kv_from") is None:
                put(p + "mix.k", (G * D, W), W ** -0.5)
                put(p + "mix.v", (G * V, W), W ** -0.5)
            put(p + "mix.g", (H, W), W ** -0.5)
            put(p + "mix.o", (W, H * V), (H * V) ** -0.5)
        elif layer["type"] == "lightning":
            for n, rows in (("q", H * D), ("k", H * D), ("v", H * V), ("g", H * V)):
                put(f"{p}mix.{n}", (rows, W), W ** -0.5)
            put(p + "mix.norm", (H * V,), 0.1, 1.0)
            put(p + "mix.o", (W, H * V), (H * V) ** -0.5)
        else:
            R, Q, Rr = m["kv_rank"], m["q_rank"], m["rot_dim"]
            put(p + "mix.dq", (Q, W), W ** -0.5)
            put(p + "mix.dq.norm", (Q,), 0.1, 1.0)
            put(p + "mix.uq", (H * (D + Rr), Q), peaky * Q ** -0.5)
            put(p + "mix.dkv", (R + Rr, W), W ** -0.5)
            put(p + "mix.dkv.norm", (R,), 0.1, 1.0)
            put(p + "mix.uk", (H * D, R), R ** -0.5)
            put(p + "mix.uv", (H * V, R), R ** -0.5)
            put(p + "mix.o", (W, H * V), (H * V) ** -0.5)
        f = layer["mlp"]
        if f is not None:
            for n in ("norm2", "norm2b"):
                put(p + n, (W,), 0.1, 1.0)
            if f["kind"] == "dense":
                put(p + "mlp.gate", (f["ff"], W), W ** -0.5)
                put(p + "mlp.up", (f["ff"], W), W ** -0.5)
                put(p + "mlp.down", (W, f["ff"]), f["ff"] ** -0.5)
            else:
                ff = f["expert"]["ff"]
                for e in range(f["router"]["experts"]):
                    put(f"{p}mlp.e{e}.gate", (ff, W), 2.0 * W ** -0.5)      # wide enough for the limit to bite
                    put(f"{p}mlp.e{e}.up", (ff, W), 2.0 * W ** -0.5)
                    put(f"{p}mlp.e{e}.down", (W, ff), ff ** -0.5)
                put(p + "mlp.router", (f["router"]["experts"], W), 1.0)      # logits far apart: a choice does not hang on rounding
                put(p + "mlp.router.b", (f["router"]["experts"],), 1.0)
    put("final.norm", (W,), 0.1, 1.0)
    put("head", (cfg["vocab"], W), W ** -0.5)
    return out


def write_folder(path: str, cfg: dict, w: dict[str, np.ndarray]) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: torch.tensor(v, dtype=torch.float64).to(torch.bfloat16).contiguous() for k, v in w.items()},
              os.path.join(path, "model.safetensors"))
    return path


def tokens(cfg: dict, n: int, seed: int) -> list[int]:
    return np.random.default_rng(1000 + seed).integers(0, cfg["vocab"], n).tolist()
