"""Bosalix: a small decoder-only design whose layers are listed one by one in config.json.

What is specific to the design and lives here: the keys of its config.json, its tensor names, which part serves which
kind of layer.  The mechanisms themselves are parts with their constants as arguments (``parts/``): a norm on every part's
output only, with weights stored around zero and a factor on what it lets into the stream (``outnorm`` blocks over
``rmsnorm`` with ``offset`` and ``mult``); a mixer input blended token by token with the row before (``token_shift``);
attention over one compressed row per position with a latent for the queries, a rotated key part that all heads share,
rotated in neighbouring pairs, and a window; attention with grouped heads, biases, a norm of every query and key head,
partial rotation in halves stretched by wavelength, unit values mixed with an earlier layer's, sigmoid weights with a bias
per head instead of a softmax, and a window that keeps the sequence's first positions in sight; routed experts of two
matrices chosen by corrected softmax scores, some of them the identity; an embedding multiplied by a constant.

config.json: ``architecture`` "Bosalix", ``vocab``, ``width``, ``norm.eps``, ``residual_mult`` (absent: 1),
``embedding.scale`` (absent: 1) and ``layers``, a list whose entries give ``type`` ("latent_attention" or "attention"),
the mixer's sizes and constants (``mixer``) and the feed-forward (``mlp``: ``kind`` "moe" with ``router.experts``,
``router.identity`` (absent: 0), ``router.top`` and ``expert.ff``; null for a layer without one).  ``rot`` holds ``dims``,
``base`` and, for attention, optionally ``scaling`` (``factor``, ``low``, ``high``, ``original``); ``mask.size`` the window
(absent: none) and ``mask.keep_first`` the first positions that stay visible (absent: 0); ``v_mix`` true marks the
attention layers whose values are mixed: the first of them is the source of the others.  Layer i's tensors are named
``l<i>.*``; a linear weight is stored [out, in].
"""
from __future__ import annotations

from dataclasses import dataclass, field

from ..config.base import ConfigError, KeyReader, require
from ..config.plan import LayerSpec, ModelPlan, PartSpec, ScheduleEntry, Source
from ..config.registry import Architecture, register_architecture

ARCHITECTURE = "Bosalix"
LATENT, ATTENTION = "latent_attention", "attention"
MAX_POSITIONS = 1 << 24         # the design names no bound of its own: the cache's size is the bound
EXPERT_ACTIVATION = "gelu"      # the erf form: fixed by the design
NORM_OFFSET = 1.0               # norm weights are stored around zero: fixed by the design


@dataclass
class Rotation:
    dims: int
    base: float
    scaling: tuple[float, float, float, float] | None = None      # factor, original, low, high


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
    window: int | None


@dataclass
class AttentionMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Rotation | None
    window: int | None
    keep_first: int = 0
    v_mix: bool = False


@dataclass
class ExpertsFfn:
    experts: int
    identity: int
    top: int
    ff: int


@dataclass
class BosalixLayer:
    type: str
    mixer: LatentMixer | AttentionMixer
    mlp: ExpertsFfn | None


@dataclass
class BosalixConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float = 1.0
    embedding_scale: float = 1.0
    layers: list[BosalixLayer] = field(default_factory=list)


def _object(data: dict, key: str, where: str, optional: bool = False) -> dict | None:
    v = data.get(key)
    if v is None and optional:
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key {key!r} must be an object, got {v!r}")
    return v


def _rotation(m: dict, where: str, width: int, may_scale: bool) -> Rotation | None:
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
    require(may_scale, f"{where}.rot: this kind of layer has no scaling of its rotation")
    s = KeyReader(scaling, where + ".rot.scaling")
    factor, original, low, high = s.number("factor"), s.number("original"), s.number("low"), s.number("high")
    require(min(factor, original, low) > 0 and high > low,
            f"{where}.rot.scaling: factor, original and low must be positive, and high above low")
    return Rotation(dims, base, (float(factor), float(original), float(low), float(high)))


def _window(m: dict, where: str) -> tuple[int | None, int]:
    mask = _object(m, "mask", where, optional=True)
    if mask is None:
        return None, 0
    r = KeyReader(mask, where + ".mask")
    size = r.integer("size", minimum=1) if mask.get("size") is not None else None
    keep = r.integer("keep_first", minimum=0) if mask.get("keep_first") is not None else 0
    return size, keep


def _mixer(kind: str, m: dict, where: str):
    r = KeyReader(m, where)
    heads = r.integer("heads", minimum=1)
    dim, vdim = r.integer("dim", minimum=1), r.integer("vdim", minimum=1)
    window, keep = _window(m, where)
    if kind == LATENT:
        require(keep == 0, f"{where}: a latent attention keeps no first positions in sight")
        rot_dim = r.integer("rot_dim", minimum=0)
        rot = _rotation(m, where, rot_dim, may_scale=False) if rot_dim else None
        require(rot_dim == 0 or (rot is not None and rot.dims == rot_dim),
                f"{where}: the rotated part has {rot_dim} numbers, rot.dims must be the same")
        return LatentMixer(heads, dim, rot_dim, vdim, r.integer("kv_rank", minimum=1), r.integer("q_rank", minimum=1),
                           r.number("scale"), rot, window)
    kv = r.integer("kv_heads", minimum=1)
    require(heads % kv == 0, f"{where}: heads {heads} is not a multiple of kv_heads {kv}")
    v_mix = m.get("v_mix", False)
    require(isinstance(v_mix, bool), f"{where}: v_mix must be true or false, got {v_mix!r}")
    return AttentionMixer(heads, kv, dim, vdim, r.number("scale"), _rotation(m, where, dim, may_scale=True), window, keep, v_mix)


def _mlp(f: dict | None, where: str) -> ExpertsFfn | None:
    if f is None:
        return None
    kind = f.get("kind")
    require(kind == "moe", f"{where}: feed-forward kind {kind!r} is not implemented (moe is)")
    router = _object(f, "router", where)
    rr = KeyReader(router, where + ".router")
    experts, top = rr.integer("experts", minimum=1), rr.integer("top", minimum=1)
    identity = rr.integer("identity", minimum=0) if router.get("identity") is not None else 0
    require(top <= experts + identity, f"{where}: top {top} exceeds the router's {experts + identity} outputs")
    return ExpertsFfn(experts, identity, top, KeyReader(_object(f, "expert", where), where + ".expert").integer("ff", minimum=1))


def config_from_json(data: dict) -> BosalixConfig:
    r = KeyReader(data)
    cfg = BosalixConfig(vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                        eps=KeyReader(_object(data, "norm", "config.json"), "config.json: norm").number("eps"))
    require(cfg.eps > 0, "norm.eps must be positive")
    if data.get("residual_mult") is not None:
        cfg.residual_mult = float(r.number("residual_mult"))
    emb = _object(data, "embedding", "config.json", optional=True)
    if emb is not None and emb.get("scale") is not None:
        cfg.embedding_scale = KeyReader(emb, "config.json: embedding").number("scale")
    layers = data.get("layers")
    require(isinstance(layers, list) and layers, "key 'layers' must be a list with at least one layer")
    for i, entry in enumerate(layers):
        where = f"config.json: layers[{i}]"
        require(isinstance(entry, dict), f"layers[{i}] must be an object")
        kind = entry.get("type")
        require(kind in (LATENT, ATTENTION), f"layers[{i}].type {kind!r} is not implemented ({LATENT} and {ATTENTION} are)")
        cfg.layers.append(BosalixLayer(kind, _mixer(kind, _object(entry, "mixer", where), where + ".mixer"),
                                       _mlp(_object(entry, "mlp", where, optional=True), where + ".mlp")))
    source = None       # the first layer whose values are mixed gives them to the others: they must be laid out alike
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, AttentionMixer) and m.v_mix:
            if source is None:
                source = m
            else:
                require((m.kv_heads, m.vdim) == (source.kv_heads, source.vdim),
                        f"layers[{i}] mixes its values with those of the first such layer, but their head counts or sizes differ")
    return cfg


def _rot_json(rot: Rotation | None) -> dict | None:
    if rot is None:
        return None
    out = {"dims": rot.dims, "base": rot.base}
    if rot.scaling is not None:
        out["scaling"] = dict(zip(("factor", "original", "low", "high"), rot.scaling))
    return out


def config_to_json(c: BosalixConfig) -> dict:
    layers = []
    for layer in c.layers:
        m = layer.mixer
        mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
        if m.rot is not None:
            mixer["rot"] = _rot_json(m.rot)
        if isinstance(m, LatentMixer):
            mixer.update({"rot_dim": m.rot_dim, "kv_rank": m.kv_rank, "q_rank": m.q_rank})
            if m.window is not None:
                mixer["mask"] = {"size": m.window}
        else:
            mixer["kv_heads"] = m.kv_heads
            if m.window is not None or m.keep_first:
                mixer["mask"] = ({} if m.window is None else {"size": m.window}) | ({"keep_first": m.keep_first} if m.keep_first else {})
            if m.v_mix:
                mixer["v_mix"] = True
        f = layer.mlp
        mlp = None if f is None else {"kind": "moe", "router": {"experts": f.experts, "identity": f.identity, "top": f.top},
                                      "expert": {"ff": f.ff}}
        layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
    return {"architecture": ARCHITECTURE, "vocab": c.vocab, "width": c.width, "norm": {"eps": c.eps},
            "residual_mult": c.residual_mult, "embedding": {"scale": c.embedding_scale}, "layers": layers}


def _position(rot: Rotation | None, head_dim: int, pairing: str) -> PartSpec:
    if rot is None:
        return PartSpec(kind="none")
    args = dict(head_dim=head_dim, rotary_dim=rot.dims, theta=rot.base, pairing=pairing)
    if rot.scaling is None:
        return PartSpec(kind="rope", args=dict(args, double_table=True))
    factor, original, low, high = rot.scaling
    return PartSpec(kind="llama3_rope", args=dict(args, factor=factor, original=original, low=low, high=high))


def plan(c: BosalixConfig) -> ModelPlan:
    def norm(name: str, mult: float) -> PartSpec:
        return PartSpec(kind="rmsnorm", args=dict(size=c.width, eps=c.eps, offset=NORM_OFFSET, mult=mult),
                        tensors={"weight": Source.single(name)})

    layers, schedule = [], []
    mix_source = None
    for i, layer in enumerate(c.layers):
        p, m = f"l{i}.mix.", layer.mixer
        if isinstance(m, LatentMixer):
            mixer = PartSpec(
                kind="latent_attention",
                args=dict(hidden_size=c.width, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, kv_rank=m.kv_rank,
                          scale=m.scale, eps=c.eps, gate_activation=None, q_rank=m.q_rank, rot_dim=m.rot_dim, window=m.window,
                          position=_position(m.rot, m.rot_dim, "interleaved") if m.rot_dim else None),
                tensors={"dq_weight": Source.single(p + "dq"), "dq_norm": Source.single(p + "dq.norm"),
                         "uq_weight": Source.single(p + "uq"), "dkv_weight": Source.single(p + "dkv"),
                         "dkv_norm": Source.single(p + "dkv.norm"), "uk_weight": Source.single(p + "uk"),
                         "uv_weight": Source.single(p + "uv"), "out_weight": Source.single(p + "o")})
        else:
            role = None
            if m.v_mix:
                role = "source" if mix_source is None else "mix"
                mix_source = i if mix_source is None else mix_source
            tensors = {"q_weight": Source.single(p + "q"), "k_weight": Source.single(p + "k"), "v_weight": Source.single(p + "v"),
                       "q_bias": Source.single(p + "q.b"), "k_bias": Source.single(p + "k.b"), "v_bias": Source.single(p + "v.b"),
                       "q_norm": Source.single(p + "q.norm"), "k_norm": Source.single(p + "k.norm"),
                       "score_bias": Source.single(p + "pb"), "out_weight": Source.single(p + "o"),
                       "out_bias": Source.single(p + "o.b")}
            if role is not None:
                tensors["mix"] = Source.single(p + "vmix")
            mixer = PartSpec(
                kind="gqa_attention",
                args=dict(hidden_size=c.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
                          scale=m.scale, window=m.window, separate_qkv=True, qkv_bias=True, out_bias=True, qk_norm_eps=c.eps,
                          value_norm_eps=c.eps, value_mix=role, sigmoid_bias=True, keep_first=m.keep_first,
                          position=_position(m.rot, m.dim, "half")),
                tensors=tensors)
        parts = {"mixer": mixer, "mixer_norm": norm(f"l{i}.norm1", c.residual_mult),
                 "mixer_shift": PartSpec(kind="token_shift", args=dict(size=c.width), tensors={"weight": Source.single(f"l{i}.shift")})}
        f = layer.mlp
        if f is not None:
            q = f"l{i}.mlp."
            E = range(f.experts)
            parts["ffn"] = PartSpec(
                kind="moe_swiglu",
                args=dict(hidden_size=c.width, num_experts=f.experts, top_k=f.top, expert_size=f.ff, shared_size=0,
                          renormalize=False, activation=EXPERT_ACTIVATION, gated=False, score_correction=True,
                          identity=f.identity),
                tensors={"router": Source.single(q + "router"), "correction": Source.single(q + "correction"),
                         "expert_up": Source.stack([f"{q}e{e}.up" for e in E]),
                         "expert_down": Source.stack([f"{q}e{e}.down" for e in E])})
            parts["ffn_norm"] = norm(f"l{i}.norm2", c.residual_mult)
        layers.append(LayerSpec(block="outnorm", parts=parts))
        schedule.append(ScheduleEntry(layer=i))
    return ModelPlan(
        architecture=ARCHITECTURE,
        vocab_size=c.vocab,
        hidden_size=c.width,
        layers=layers,
        schedule=schedule,
        final_norm=norm("final.norm", 1.0),
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
