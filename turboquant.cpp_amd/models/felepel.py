"""Felepel: a small decoder-only design whose layers are listed one by one in config.json.

What is specific to the design and lives here: the keys of its config.json, its tensor names, which part serves which
kind of layer.  The mechanisms themselves are parts with their constants as arguments (``parts/``): attention with
capped scores, a bias by distance and chunks of positions; the gated delta rule with a decay per key channel;
experts chosen within the best groups; a norm before and after every part; a learned vector per position.

config.json: ``architecture`` "Felepel", ``vocab``, ``width``, ``max_positions``, ``norm.eps`` and ``layers``, a list
whose entries give ``type`` ("attention" or "channel_delta"), the mixer's sizes and constants (``mixer``), the
feed-forward (``mlp``, null for a layer without one) and optionally ``weights_of``: j, for a layer that runs layer j's
tensors with a cache or state of its own.  Layer i's tensors are named ``l<i>.*``; a linear weight is stored
[out, in].  The ranks of the delta rule's two low-rank products are not in config.json: they are the shapes of
``mix.a1`` and ``mix.g1`` (``complete``), or the keys ``decay_rank`` / ``gate_rank`` that this library writes into the
mixer's object of a folder it makes itself.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field

from ..config.base import ConfigError, KeyReader, require
from ..config.plan import LayerSpec, ModelPlan, PartSpec, ScheduleEntry, Source
from ..config.registry import Architecture, register_architecture

ARCHITECTURE = "Felepel"
ATTENTION, DELTA = "attention", "channel_delta"


@dataclass
class AttentionMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float | None       # None: scores are not capped
    chunk: int | None           # None: every earlier position is seen


@dataclass
class DeltaMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int                   # taps of the short convolution
    decay_rank: int | None      # None until the checkpoint's shapes have been seen
    gate_rank: int | None


@dataclass
class ExpertsFfn:
    experts: int
    top: int
    ff: int
    groups: int                 # 1: the choice is among all experts
    keep: int


@dataclass
class FelepelLayer:
    type: str
    mixer: AttentionMixer | DeltaMixer
    mlp: ExpertsFfn | None
    weights_of: int | None = None


@dataclass
class FelepelConfig:
    vocab: int
    width: int
    max_positions: int
    eps: float
    layers: list[FelepelLayer] = field(default_factory=list)


def _object(data: dict, key: str, where: str, optional: bool = False) -> dict | None:
    v = data.get(key)
    if v is None and optional:
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key {key!r} must be an object, got {v!r}")
    return v


def _mixer(kind: str, m: dict, where: str):
    r = KeyReader(m, where)
    heads, kv = r.integer("heads", minimum=1), r.integer("kv_heads", minimum=1)
    require(heads % kv == 0, f"{where}: heads {heads} is not a multiple of kv_heads {kv}")
    dim, vdim = r.integer("dim", minimum=1), r.integer("vdim", minimum=1)
    if kind == ATTENTION:
        mask = _object(m, "mask", where, optional=True)
        chunk = KeyReader(mask, where + ".mask").integer("size", minimum=1) if mask is not None else None
        cap = m.get("softcap")
        cap = None if cap is None else r.number("softcap")
        require(cap is None or cap > 0, f"{where}: softcap must be positive")
        return AttentionMixer(heads, kv, dim, vdim, r.number("scale"), cap, chunk)
    return DeltaMixer(heads, kv, dim, vdim, r.integer("conv", minimum=1), r.optional_integer("decay_rank"),
                      r.optional_integer("gate_rank"))


def _mlp(f: dict | None, where: str) -> ExpertsFfn | None:
    if f is None:
        return None
    kind = f.get("kind")
    require(kind == "moe", f"{where}: feed-forward kind {kind!r} is not implemented (moe is)")
    router = KeyReader(_object(f, "router", where), where + ".router")
    experts, top = router.integer("experts", minimum=1), router.integer("top", minimum=1)
    require(top <= experts, f"{where}: top {top} exceeds experts {experts}")
    groups = _object(router.data, "groups", where + ".router", optional=True)
    count, keep = 1, 1
    if groups is not None:
        g = KeyReader(groups, where + ".router.groups")
        count, keep = g.integer("count", minimum=1), g.integer("keep", minimum=1)
        require(experts % count == 0 and keep <= count and top <= keep * (experts // count),
                f"{where}: {count} groups of which {keep} are kept do not fit {experts} experts with {top} per token")
    ff = KeyReader(_object(f, "expert", where), where + ".expert").integer("ff", minimum=1)
    return ExpertsFfn(experts, top, ff, count, keep)


def config_from_json(data: dict) -> FelepelConfig:
    r = KeyReader(data)
    cfg = FelepelConfig(vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                        max_positions=r.integer("max_positions", minimum=1),
                        eps=KeyReader(_object(data, "norm", "config.json"), "config.json: norm").number("eps"))
    require(cfg.eps > 0, "norm.eps must be positive")
    layers = data.get("layers")
    require(isinstance(layers, list) and layers, "key 'layers' must be a list with at least one layer")
    for i, entry in enumerate(layers):
        where = f"config.json: layers[{i}]"
        require(isinstance(entry, dict), f"layers[{i}] must be an object")
        kind = entry.get("type")
        require(kind in (ATTENTION, DELTA), f"layers[{i}].type {kind!r} is not implemented ({ATTENTION} and {DELTA} are)")
        of = entry.get("weights_of")
        require(of is None or (isinstance(of, int) and not isinstance(of, bool) and 0 <= of < len(layers) and of != i),
                f"layers[{i}].weights_of must name another layer, got {of!r}")
        cfg.layers.append(FelepelLayer(kind, _mixer(kind, _object(entry, "mixer", where), where + ".mixer"),
                                       _mlp(_object(entry, "mlp", where, optional=True), where + ".mlp"), of))
    for i, layer in enumerate(cfg.layers):      # a layer on another's tensors: the other has its own, and the two agree
        of = layer.weights_of
        if of is None:
            continue
        src = cfg.layers[of]
        require(src.weights_of is None, f"layers[{i}].weights_of names layer {of}, which has no tensors of its own")
        require(src.type == layer.type, f"layers[{i}] is {layer.type} but uses the weights of layer {of}, which is {src.type}")
        if isinstance(layer.mixer, DeltaMixer):     # the ranks are the tensors' and so the other layer's
            layer.mixer.decay_rank, layer.mixer.gate_rank = src.mixer.decay_rank, src.mixer.gate_rank
        require(layer.mixer == src.mixer and layer.mlp == src.mlp,
                f"layers[{i}] uses the weights of layer {of} but its sizes or constants differ")
    return cfg


def complete(cfg: FelepelConfig, shapes: dict) -> FelepelConfig:
    """The sizes that only the checkpoint's tensors give: the ranks of the delta rule's low-rank products, and how many
    positions the table of learned position vectors has if that is not what config.json says."""
    cfg = copy.deepcopy(cfg)
    if "pos" in shapes and len(shapes["pos"]) == 2:
        cfg.max_positions = int(shapes["pos"][0])
    for i, layer in enumerate(cfg.layers):
        if not isinstance(layer.mixer, DeltaMixer):
            continue
        p = f"l{i if layer.weights_of is None else layer.weights_of}.mix."
        for attr, name in (("decay_rank", p + "a1"), ("gate_rank", p + "g1")):
            if name in shapes and len(shapes[name]) == 2:
                have = getattr(layer.mixer, attr)
                if have is not None and have != shapes[name][0]:
                    raise ConfigError(f"config.json: layers[{i}].mixer.{attr} is {have}, tensor {name} has {shapes[name][0]} rows")
                setattr(layer.mixer, attr, int(shapes[name][0]))
    return cfg


def config_to_json(c: FelepelConfig) -> dict:
    layers = []
    for layer in c.layers:
        m = layer.mixer
        mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim}
        if isinstance(m, AttentionMixer):
            mixer["scale"] = m.scale
            if m.softcap is not None:
                mixer["softcap"] = m.softcap
            if m.chunk is not None:
                mixer["mask"] = {"size": m.chunk}
        else:
            mixer["conv"] = m.conv
            if m.decay_rank is not None:
                mixer["decay_rank"], mixer["gate_rank"] = m.decay_rank, m.gate_rank
        f = layer.mlp
        mlp = None if f is None else {"kind": "moe", "expert": {"ff": f.ff},
                                      "router": {"experts": f.experts, "top": f.top,
                                                 "groups": {"count": f.groups, "keep": f.keep}}}
        entry = {"type": layer.type, "mixer": mixer, "mlp": mlp}
        if layer.weights_of is not None:
            entry["weights_of"] = layer.weights_of
        layers.append(entry)
    return {"architecture": ARCHITECTURE, "vocab": c.vocab, "width": c.width, "max_positions": c.max_positions,
            "norm": {"eps": c.eps}, "layers": layers}


def plan(c: FelepelConfig) -> ModelPlan:
    def norm(name: str) -> PartSpec:
        return PartSpec(kind="rmsnorm", args=dict(size=c.width, eps=c.eps), tensors={"weight": Source.single(name)})

    layers, layer_of = [], {}
    for i, layer in enumerate(c.layers):
        if layer.weights_of is not None:
            continue
        layer_of[i] = len(layers)
        p, m = f"l{i}.", layer.mixer
        if isinstance(m, AttentionMixer):
            mixer = PartSpec(
                kind="gqa_attention",
                args=dict(hidden_size=c.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim,
                          value_dim=m.vdim, qkv_bias=True, out_bias=True, scale=m.scale, score_cap=m.softcap,
                          distance_bias=True, chunk=m.chunk, separate_qkv=True, position=PartSpec(kind="none")),
                tensors={"q_weight": Source.single(p + "mix.q"), "k_weight": Source.single(p + "mix.k"),
                         "v_weight": Source.single(p + "mix.v"), "out_weight": Source.single(p + "mix.o"),
                         "q_bias": Source.single(p + "mix.q.b"), "k_bias": Source.single(p + "mix.k.b"),
                         "v_bias": Source.single(p + "mix.v.b"), "out_bias": Source.single(p + "mix.o.b"),
                         "r1": Source.single(p + "mix.r1"), "r2": Source.single(p + "mix.r2")})
        else:
            if m.decay_rank is None or m.gate_rank is None:
                raise ConfigError(f"config.json: layers[{i}].mixer: the ranks of the decay's and the gate's products are "
                                  "known from the checkpoint's tensors only (or from decay_rank / gate_rank)")
            mixer = PartSpec(
                kind="channel_delta",
                args=dict(hidden_size=c.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim,
                          value_dim=m.vdim, conv_taps=m.conv, rank_a=m.decay_rank, rank_g=m.gate_rank, eps=c.eps),
                tensors={"q_weight": Source.single(p + "mix.q"), "k_weight": Source.single(p + "mix.k"),
                         "v_weight": Source.single(p + "mix.v"), "q_conv": Source.single(p + "mix.q.conv"),
                         "k_conv": Source.single(p + "mix.k.conv"), "v_conv": Source.single(p + "mix.v.conv"),
                         "b_weight": Source.single(p + "mix.b"), "a1_weight": Source.single(p + "mix.a1"),
                         "a2_weight": Source.single(p + "mix.a2"), "g1_weight": Source.single(p + "mix.g1"),
                         "g2_weight": Source.single(p + "mix.g2"), "a_log": Source.single(p + "mix.A_log"),
                         "dt_bias": Source.single(p + "mix.dt_bias"), "out_norm": Source.single(p + "mix.norm"),
                         "out_weight": Source.single(p + "mix.o")})
        parts = {"mixer_norm": norm(p + "norm1"), "mixer": mixer, "mixer_post_norm": norm(p + "norm1b")}
        f = layer.mlp
        if f is not None:
            E = range(f.experts)
            parts.update({
                "ffn_norm": norm(p + "norm2"),
                "ffn": PartSpec(
                    kind="moe_swiglu",
                    args=dict(hidden_size=c.width, num_experts=f.experts, top_k=f.top, expert_size=f.ff, shared_size=0,
                              renormalize=False, groups=(f.groups, f.keep)),
                    tensors={"router": Source.single(p + "mlp.router"),
                             "expert_gate": Source.stack([f"{p}mlp.e{e}.gate" for e in E]),
                             "expert_up": Source.stack([f"{p}mlp.e{e}.up" for e in E]),
                             "expert_down": Source.stack([f"{p}mlp.e{e}.down" for e in E])}),
                "ffn_post_norm": norm(p + "norm2b"),
            })
        layers.append(LayerSpec(block="sandwich", parts=parts))
    # a layer that names another's weights is one more run of that layer, with a cache or state of its own
    schedule = [ScheduleEntry(layer=layer_of[i if layer.weights_of is None else layer.weights_of])
                for i, layer in enumerate(c.layers)]
    return ModelPlan(
        architecture=ARCHITECTURE,
        vocab_size=c.vocab,
        hidden_size=c.width,
        layers=layers,
        schedule=schedule,
        final_norm=norm("final.norm"),
        embedding=Source.single("embed"),
        lm_head=Source.single("head"),
        max_positions=c.max_positions,
        position_table=Source.single("pos"),
    )


register_architecture(Architecture(
    name=ARCHITECTURE,
    config_from_json=config_from_json,
    plan=plan,
    config_to_json=config_to_json,
    complete=complete,
))
