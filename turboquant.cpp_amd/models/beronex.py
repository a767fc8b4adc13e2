"""Beronex: a small decoder-only design whose layers are listed one by one in config.json.

What is specific to the design and lives here: the keys of its config.json, its tensor names, which part serves which
kind of layer.  The mechanisms themselves are parts with their constants as arguments (``parts/``): a norm before and
after every part (``sandwich`` blocks); linear attention with a constant decay per head; attention over one compressed
row per position with a latent for the queries and a rotated key part that all heads share; attention with grouped heads,
rotation in neighbouring pairs, a norm of every query and key head behind the rotation, a window, a gate per head, and
layers that read another layer's keys and values; rotations stretched by YaRN; a dense gated feed-forward and one of
routed experts whose pairs are clamped; an embedding multiplied by a constant.

config.json: ``architecture`` "Beronex", ``vocab``, ``width``, ``norm.eps``, ``embedding.scale`` (absent: 1) and
``layers``, a list whose entries give ``type`` ("lightning", "latent_attention" or "attention"), the mixer's sizes and
constants (``mixer``) and the feed-forward (``mlp``: ``kind`` "dense" with ``ff``, or "moe" with ``router.experts``,
``router.top``, ``expert.ff`` and ``expert.limit``; null for a layer without one).  ``rot`` holds ``dims``, ``base`` and,
optionally, ``scaling`` (``factor``, ``original``, ``fast``, ``slow``); ``mask.size`` the window (absent: none).  An
attention with ``kv_from``: j has no key and value matrices and reads the keys and values that layer j keeps.  Layer i's
tensors are named ``l<i>.*``; a linear weight is stored [out, in].
"""
from __future__ import annotations

from dataclasses import dataclass, field

from ..config.base import ConfigError, KeyReader, require
from ..config.plan import LayerSpec, ModelPlan, PartSpec, ScheduleEntry, Source
from ..config.registry import Architecture, register_architecture

ARCHITECTURE = "Beronex"
LIGHTNING, LATENT, ATTENTION = "lightning", "latent_attention", "attention"
MAX_POSITIONS = 1 << 24         # the design names no bound of its own: the cache's size is the bound
EXPERT_ACTIVATION = "swish1702"  # g sigmoid(1.702 g): fixed by the design


@dataclass
class Rotation:
    dims: int
    base: float
    scaling: tuple[float, float, float, float] | None = None      # factor, original, fast, slow


@dataclass
class LightningMixer:
    heads: int
    dim: int
    vdim: int
    decay: list[float]


@dataclass
class LatentMixer:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: Rotation | None


@dataclass
class AttentionMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Rotation | None
    window: int | None
    kv_from: int | None = None


@dataclass
class DenseFfn:
    ff: int


@dataclass
class ExpertsFfn:
    experts: int
    top: int
    ff: int
    limit: float


@dataclass
class BeronexLayer:
    type: str
    mixer: LightningMixer | LatentMixer | AttentionMixer
    mlp: DenseFfn | ExpertsFfn | None


@dataclass
class BeronexConfig:
    vocab: int
    width: int
    eps: float
    embedding_scale: float = 1.0
    layers: list[BeronexLayer] = field(default_factory=list)


def _object(data: dict, key: str, where: str, optional: bool = False) -> dict | None:
    v = data.get(key)
    if v is None and optional:
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key {key!r} must be an object, got {v!r}")
    return v


def _rotation(m: dict, where: str, width: int) -> Rotation | None:
    rot = _object(m, "rot", where, optional=True)
    if rot is None:
        return None
    r = KeyReader(rot, where + ".rot")
    dims, base = r.integer("dims", minimum=0), r.number("base")
    require(dims % 2 == 0 and dims <= width, f"{where}.rot: dims {dims} must be even and at most {width}")
    require(base > 0, f"{where}.rot: base must be positive")
    if dims == 0:
        return None
    scaling = _object(rot, "scaling", where + ".rot", optional=True)
    if scaling is None:
        return Rotation(dims, base)
    s = KeyReader(scaling, where + ".rot.scaling")
    values = (s.number("factor"), s.number("original"), s.number("fast"), s.number("slow"))
    require(min(values) > 0 and base != 1,
            f"{where}.rot.scaling: factor, original, fast and slow must be positive, and base other than 1")
    return Rotation(dims, base, tuple(float(v) for v in values))


def _mixer(kind: str, m: dict, where: str, index: int, n_layers: int):
    r = KeyReader(m, where)
    heads = r.integer("heads", minimum=1)
    dim, vdim = r.integer("dim", minimum=1), r.integer("vdim", minimum=1)
    if kind == LIGHTNING:
        decay = m.get("decay")
        if isinstance(decay, (int, float)) and not isinstance(decay, bool):      # one number: the same for every head
            decay = [decay] * heads
        require(isinstance(decay, list) and len(decay) == heads
                and all(isinstance(d, (int, float)) and not isinstance(d, bool) and 0 <= d <= 1 for d in decay),
                f"{where}: decay must list a number between 0 and 1 for each of the {heads} heads")
        return LightningMixer(heads, dim, vdim, [float(d) for d in decay])
    if kind == LATENT:
        rot_dim = r.integer("rot_dim", minimum=0)
        rot = _rotation(m, where, rot_dim) if rot_dim else None
        require(rot_dim == 0 or (rot is not None and rot.dims == rot_dim),
                f"{where}: the rotated part has {rot_dim} numbers, rot.dims must be the same")
        return LatentMixer(heads, dim, rot_dim, vdim, r.integer("kv_rank", minimum=1), r.integer("q_rank", minimum=1),
                           r.number("scale"), rot)
    kv = r.integer("kv_heads", minimum=1)
    require(heads % kv == 0, f"{where}: heads {heads} is not a multiple of kv_heads {kv}")
    mask = _object(m, "mask", where, optional=True)
    window = KeyReader(mask, where + ".mask").integer("size", minimum=1) if mask is not None else None
    of = m.get("kv_from")
    require(of is None or (isinstance(of, int) and not isinstance(of, bool) and 0 <= of < n_layers and of != index),
            f"{where}: kv_from must name another layer, got {of!r}")
    return AttentionMixer(heads, kv, dim, vdim, r.number("scale"), _rotation(m, where, dim), window, of)


def _mlp(f: dict | None, where: str) -> DenseFfn | ExpertsFfn | None:
    if f is None:
        return None
    kind = f.get("kind")
    require(kind in ("dense", "moe"), f"{where}: feed-forward kind {kind!r} is not implemented (dense and moe are)")
    if kind == "dense":
        return DenseFfn(KeyReader(f, where).integer("ff", minimum=1))
    router = KeyReader(_object(f, "router", where), where + ".router")
    experts, top = router.integer("experts", minimum=1), router.integer("top", minimum=1)
    require(top <= experts, f"{where}: top {top} exceeds experts {experts}")
    e = KeyReader(_object(f, "expert", where), where + ".expert")
    limit = e.number("limit")
    require(limit > 0, f"{where}.expert: limit must be positive")
    return ExpertsFfn(experts, top, e.integer("ff", minimum=1), limit)


def config_from_json(data: dict) -> BeronexConfig:
    r = KeyReader(data)
    cfg = BeronexConfig(vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                        eps=KeyReader(_object(data, "norm", "config.json"), "config.json: norm").number("eps"))
    require(cfg.eps > 0, "norm.eps must be positive")
    emb = _object(data, "embedding", "config.json", optional=True)
    if emb is not None and emb.get("scale") is not None:
        cfg.embedding_scale = KeyReader(emb, "config.json: embedding").number("scale")
    layers = data.get("layers")
    require(isinstance(layers, list) and layers, "key 'layers' must be a list with at least one layer")
    for i, entry in enumerate(layers):
        where = f"config.json: layers[{i}]"
        require(isinstance(entry, dict), f"layers[{i}] must be an object")
        kind = entry.get("type")
        require(kind in (LIGHTNING, LATENT, ATTENTION),
                f"layers[{i}].type {kind!r} is not implemented ({LIGHTNING}, {LATENT} and {ATTENTION} are)")
        cfg.layers.append(BeronexLayer(kind, _mixer(kind, _object(entry, "mixer", where), where + ".mixer", i, len(layers)),
                                       _mlp(_object(entry, "mlp", where, optional=True), where + ".mlp")))
    for i, layer in enumerate(cfg.layers):      # a layer on another's keys and values: the other has its own, like this one's
        m = layer.mixer
        if not isinstance(m, AttentionMixer) or m.kv_from is None:
            continue
        src = cfg.layers[m.kv_from].mixer
        require(isinstance(src, AttentionMixer) and src.kv_from is None,
                f"layers[{i}].mixer.kv_from names layer {m.kv_from}, which keeps no keys and values of its own")
        require((src.kv_heads, src.dim, src.vdim) == (m.kv_heads, m.dim, m.vdim),
                f"layers[{i}] reads the keys and values of layer {m.kv_from} but their head counts or sizes differ")
        require(m.kv_from < i, f"layers[{i}] reads the keys and values of layer {m.kv_from}, which runs after it")
    return cfg


def _rot_json(rot: Rotation | None) -> dict | None:
    if rot is None:
        return None
    out = {"dims": rot.dims, "base": rot.base}
    if rot.scaling is not None:
        out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), rot.scaling))
    return out


def config_to_json(c: BeronexConfig) -> dict:
    layers = []
    for layer in c.layers:
        m = layer.mixer
        mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim}
        if isinstance(m, LightningMixer):
            mixer["decay"] = list(m.decay)
        elif isinstance(m, LatentMixer):
            mixer.update({"rot_dim": m.rot_dim, "kv_rank": m.kv_rank, "q_rank": m.q_rank, "scale": m.scale})
            if m.rot is not None:
                mixer["rot"] = _rot_json(m.rot)
        else:
            mixer.update({"kv_heads": m.kv_heads, "scale": m.scale})
            if m.rot is not None:
                mixer["rot"] = _rot_json(m.rot)
            if m.window is not None:
                mixer["mask"] = {"size": m.window}
            if m.kv_from is not None:
                mixer["kv_from"] = m.kv_from
        f = layer.mlp
        if f is None:
            mlp = None
        elif isinstance(f, DenseFfn):
            mlp = {"kind": "dense", "ff": f.ff}
        else:
            mlp = {"kind": "moe", "router": {"experts": f.experts, "top": f.top}, "expert": {"ff": f.ff, "limit": f.limit}}
        layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
    return {"architecture": ARCHITECTURE, "vocab": c.vocab, "width": c.width, "norm": {"eps": c.eps},
            "embedding": {"scale": c.embedding_scale}, "layers": layers}


def _position(rot: Rotation | None, head_dim: int, pairing: str) -> PartSpec:
    if rot is None:
        return PartSpec(kind="none")
    args = dict(head_dim=head_dim, rotary_dim=rot.dims, theta=rot.base, pairing=pairing)
    if rot.scaling is None:
        return PartSpec(kind="rope", args=args)
    factor, original, fast, slow = rot.scaling
    return PartSpec(kind="yarn_rope", args=dict(args, factor=factor, original=original, fast=fast, slow=slow))


def plan(c: BeronexConfig) -> ModelPlan:
    def norm(name: str) -> PartSpec:
        return PartSpec(kind="rmsnorm", args=dict(size=c.width, eps=c.eps), tensors={"weight": Source.single(name)})

    # what a layer's cache must keep: its own window, or that of a later layer that reads its keys and values if wider
    keeps: dict[int, int | None] = {}
    for i, layer in enumerate(c.layers):
        m = layer.mixer
        if isinstance(m, AttentionMixer):
            owner = i if m.kv_from is None else m.kv_from
            if owner not in keeps:
                keeps[owner] = m.window
            elif keeps[owner] is not None:
                keeps[owner] = None if m.window is None else max(keeps[owner], m.window)

    layers, schedule = [], []
    for i, layer in enumerate(c.layers):
        p, m = f"l{i}.mix.", layer.mixer
        cache_of = None
        if isinstance(m, LightningMixer):
            mixer = PartSpec(
                kind="lightning",
                args=dict(hidden_size=c.width, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, decay=list(m.decay), eps=c.eps),
                tensors={"q_weight": Source.single(p + "q"), "k_weight": Source.single(p + "k"), "v_weight": Source.single(p + "v"),
                         "g_weight": Source.single(p + "g"), "out_norm": Source.single(p + "norm"),
                         "out_weight": Source.single(p + "o")})
        elif isinstance(m, LatentMixer):
            mixer = PartSpec(
                kind="latent_attention",
                args=dict(hidden_size=c.width, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, kv_rank=m.kv_rank,
                          scale=m.scale, eps=c.eps, gate_activation=None, q_rank=m.q_rank, rot_dim=m.rot_dim,
                          position=_position(m.rot, m.rot_dim, "half") if m.rot_dim else None),
                tensors={"dq_weight": Source.single(p + "dq"), "dq_norm": Source.single(p + "dq.norm"),
                         "uq_weight": Source.single(p + "uq"), "dkv_weight": Source.single(p + "dkv"),
                         "dkv_norm": Source.single(p + "dkv.norm"), "uk_weight": Source.single(p + "uk"),
                         "uv_weight": Source.single(p + "uv"), "out_weight": Source.single(p + "o")})
        else:
            shares = m.kv_from is not None
            tensors = {"q_weight": Source.single(p + "q"), "gate_weight": Source.single(p + "g"),
                       "out_weight": Source.single(p + "o")}
            if shares:
                cache_of = m.kv_from          # schedule entry i runs layer i
            else:
                tensors.update({"k_weight": Source.single(p + "k"), "v_weight": Source.single(p + "v")})
            mixer = PartSpec(
                kind="gqa_attention",
                args=dict(hidden_size=c.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
                          scale=m.scale, window=m.window, separate_qkv=True, rotated_norm_eps=c.eps, head_gate=True,
                          shares_kv=shares, cache_window=m.window if shares else keeps[i],
                          position=_position(m.rot, m.dim, "interleaved")),
                tensors=tensors)
        parts = {"mixer_norm": norm(f"l{i}.norm1"), "mixer": mixer, "mixer_post_norm": norm(f"l{i}.norm1b")}
        f = layer.mlp
        if f is not None:
            q = f"l{i}.mlp."
            if isinstance(f, DenseFfn):
                ffn = PartSpec(kind="dense_swiglu", args=dict(hidden_size=c.width, inner_size=f.ff, activation="gelu_tanh"),
                               tensors={"gate": Source.single(q + "gate"), "up": Source.single(q + "up"),
                                        "down": Source.single(q + "down")})
            else:
                E = range(f.experts)
                ffn = PartSpec(
                    kind="moe_swiglu",
                    args=dict(hidden_size=c.width, num_experts=f.experts, top_k=f.top, expert_size=f.ff, shared_size=0,
                              renormalize=True, activation=EXPERT_ACTIVATION, router_bias=True, pair_limit=f.limit),
                    tensors={"router": Source.single(q + "router"), "router_bias": Source.single(q + "router.b"),
                             "expert_gate": Source.stack([f"{q}e{e}.gate" for e in E]),
                             "expert_up": Source.stack([f"{q}e{e}.up" for e in E]),
                             "expert_down": Source.stack([f"{q}e{e}.down" for e in E])})
            parts.update({"ffn_norm": norm(f"l{i}.norm2"), "ffn": ffn, "ffn_post_norm": norm(f"l{i}.norm2b")})
        layers.append(LayerSpec(block="sandwich", parts=parts))
        schedule.append(ScheduleEntry(layer=i, cache_of=cache_of))
    return ModelPlan(
        architecture=ARCHITECTURE,
        vocab_size=c.vocab,
        hidden_size=c.width,
        layers=layers,
        schedule=schedule,
        final_norm=norm("final.norm"),
        embedding=Source.single("embed"),
        lm_head=Source.single("head"),
        max_positions=MAX_POSITIONS,
        embedding_scale=c.embedding_scale,
    )


register_architecture(Architecture(
    name=ARCHITECTURE,
    config_from_json=config_from_json,
    plan=plan,
    config_to_json=config_to_json,
))
