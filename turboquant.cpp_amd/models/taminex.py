"""Taminex: a small decoder-only design whose layers are listed one by one in config.json.

What is specific to the design and lives here: the keys of its config.json, its tensor names, which part serves which
kind of layer.  The mechanisms themselves are parts with their constants as arguments (``parts/``): a norm on every
part's output only (``outnorm`` blocks: the parts read the residual stream itself); attention with grouped heads, biases,
a norm of every query and key head, rotation of the first dimensions of a head in neighbouring pairs and a learned sink
per head in the softmax's denominator; the gated delta rule with one decay per head; attention over one compressed row
per position that a later layer may share; a feed-forward of two matrices with the square of relu between them; tied
embeddings, logits multiplied by a constant and then capped.

config.json: ``architecture`` "Taminex", ``vocab``, ``width``, ``norm.eps``, ``logit_scale`` and ``logit_softcap``
(absent: 1 and no cap), and ``layers``, a list whose entries give ``type`` ("attention", "delta" or
"latent_attention"), the mixer's sizes and constants (``mixer``) and the feed-forward (``mlp``: ``kind`` "dense" and
``ff``; null for a layer without one).  A latent attention with ``kv_from``: j has no compression of its own and reads
the latents that layer j keeps.  Layer i's tensors are named ``l<i>.*``; a linear weight is stored [out, in].
"""
from __future__ import annotations

from dataclasses import dataclass, field

from ..config.base import ConfigError, KeyReader, require
from ..config.plan import LayerSpec, ModelPlan, PartSpec, ScheduleEntry, Source
from ..config.registry import Architecture, register_architecture

ARCHITECTURE = "Taminex"
ATTENTION, DELTA, LATENT = "attention", "delta", "latent_attention"
MAX_POSITIONS = 1 << 24         # the design names no bound of its own: the cache's size is the bound


@dataclass
class AttentionMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int               # 0: no rotation
    rot_base: float


@dataclass
class DeltaMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int                   # taps of the short convolution


@dataclass
class LatentMixer:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float
    kv_from: int | None = None  # the layer whose latents this one reads


@dataclass
class DenseFfn:
    ff: int


@dataclass
class TaminexLayer:
    type: str
    mixer: AttentionMixer | DeltaMixer | LatentMixer
    mlp: DenseFfn | None


@dataclass
class TaminexConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float = 1.0
    logit_softcap: float | None = None
    layers: list[TaminexLayer] = field(default_factory=list)


def _object(data: dict, key: str, where: str, optional: bool = False) -> dict | None:
    v = data.get(key)
    if v is None and optional:
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key {key!r} must be an object, got {v!r}")
    return v


def _mixer(kind: str, m: dict, where: str, index: int, n_layers: int):
    r = KeyReader(m, where)
    heads = r.integer("heads", minimum=1)
    dim, vdim = r.integer("dim", minimum=1), r.integer("vdim", minimum=1)
    if kind == LATENT:
        of = m.get("kv_from")
        require(of is None or (isinstance(of, int) and not isinstance(of, bool) and 0 <= of < n_layers and of != index),
                f"{where}: kv_from must name another layer, got {of!r}")
        return LatentMixer(heads, dim, vdim, r.integer("kv_rank", minimum=1), r.number("scale"), of)
    kv = r.integer("kv_heads", minimum=1)
    require(heads % kv == 0, f"{where}: heads {heads} is not a multiple of kv_heads {kv}")
    if kind == DELTA:
        return DeltaMixer(heads, kv, dim, vdim, r.integer("conv", minimum=1))
    rot = _object(m, "rot", where, optional=True)
    dims, base = 0, 10000.0
    if rot is not None:
        rr = KeyReader(rot, where + ".rot")
        dims, base = rr.integer("dims", minimum=0), rr.number("base")
        require(dims % 2 == 0 and dims <= dim, f"{where}.rot: dims {dims} must be even and at most dim {dim}")
        require(base > 0, f"{where}.rot: base must be positive")
    return AttentionMixer(heads, kv, dim, vdim, r.number("scale"), dims, base)


def _mlp(f: dict | None, where: str) -> DenseFfn | None:
    if f is None:
        return None
    kind = f.get("kind")
    require(kind == "dense", f"{where}: feed-forward kind {kind!r} is not implemented (dense is)")
    return DenseFfn(KeyReader(f, where).integer("ff", minimum=1))


def config_from_json(data: dict) -> TaminexConfig:
    r = KeyReader(data)
    cfg = TaminexConfig(vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                        eps=KeyReader(_object(data, "norm", "config.json"), "config.json: norm").number("eps"))
    require(cfg.eps > 0, "norm.eps must be positive")
    if data.get("logit_scale") is not None:
        cfg.logit_scale = r.number("logit_scale")
    if data.get("logit_softcap") is not None:
        cfg.logit_softcap = r.number("logit_softcap")
        require(cfg.logit_softcap > 0, "logit_softcap must be positive")
    layers = data.get("layers")
    require(isinstance(layers, list) and layers, "key 'layers' must be a list with at least one layer")
    for i, entry in enumerate(layers):
        where = f"config.json: layers[{i}]"
        require(isinstance(entry, dict), f"layers[{i}] must be an object")
        kind = entry.get("type")
        require(kind in (ATTENTION, DELTA, LATENT),
                f"layers[{i}].type {kind!r} is not implemented ({ATTENTION}, {DELTA} and {LATENT} are)")
        cfg.layers.append(TaminexLayer(kind, _mixer(kind, _object(entry, "mixer", where), where + ".mixer", i, len(layers)),
                                       _mlp(_object(entry, "mlp", where, optional=True), where + ".mlp")))
    for i, layer in enumerate(cfg.layers):      # a layer on another's latents: the other keeps its own, of the same size, and runs first
        m = layer.mixer
        if not isinstance(m, LatentMixer) or m.kv_from is None:
            continue
        src = cfg.layers[m.kv_from].mixer
        require(isinstance(src, LatentMixer) and src.kv_from is None,
                f"layers[{i}].mixer.kv_from names layer {m.kv_from}, which keeps no latents of its own")
        require(src.kv_rank == m.kv_rank, f"layers[{i}] reads the latents of layer {m.kv_from} but their kv_rank differ")
        require(m.kv_from < i, f"layers[{i}] reads the latents of layer {m.kv_from}, which runs after it")
    return cfg


def config_to_json(c: TaminexConfig) -> dict:
    layers = []
    for layer in c.layers:
        m = layer.mixer
        mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim}
        if isinstance(m, AttentionMixer):
            mixer.update({"kv_heads": m.kv_heads, "scale": m.scale, "rot": {"dims": m.rot_dims, "base": m.rot_base}})
        elif isinstance(m, DeltaMixer):
            mixer.update({"kv_heads": m.kv_heads, "conv": m.conv})
        else:
            mixer.update({"kv_rank": m.kv_rank, "scale": m.scale})
            if m.kv_from is not None:
                mixer["kv_from"] = m.kv_from
        layers.append({"type": layer.type, "mixer": mixer,
                       "mlp": None if layer.mlp is None else {"kind": "dense", "ff": layer.mlp.ff}})
    out = {"architecture": ARCHITECTURE, "vocab": c.vocab, "width": c.width, "norm": {"eps": c.eps},
           "logit_scale": c.logit_scale, "layers": layers}
    if c.logit_softcap is not None:
        out["logit_softcap"] = c.logit_softcap
    return out


def plan(c: TaminexConfig) -> ModelPlan:
    def norm(name: str) -> PartSpec:
        return PartSpec(kind="rmsnorm", args=dict(size=c.width, eps=c.eps), tensors={"weight": Source.single(name)})

    layers, schedule = [], []
    for i, layer in enumerate(c.layers):
        p, m = f"l{i}.mix.", layer.mixer
        cache_of = None
        if isinstance(m, AttentionMixer):
            position = PartSpec(kind="none") if m.rot_dims == 0 else \
                PartSpec(kind="rope", args=dict(head_dim=m.dim, rotary_dim=m.rot_dims, theta=m.rot_base, pairing="interleaved"))
            mixer = PartSpec(
                kind="gqa_attention",
                args=dict(hidden_size=c.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
                          qkv_bias=True, scale=m.scale, qk_norm_eps=c.eps, separate_qkv=True, sink=True, position=position),
                tensors={"q_weight": Source.single(p + "q"), "k_weight": Source.single(p + "k"),
                         "v_weight": Source.single(p + "v"), "out_weight": Source.single(p + "o"),
                         "q_bias": Source.single(p + "q.b"), "k_bias": Source.single(p + "k.b"),
                         "v_bias": Source.single(p + "v.b"), "q_norm": Source.single(p + "q.norm"),
                         "k_norm": Source.single(p + "k.norm"), "sink": Source.single(p + "sink")})
        elif isinstance(m, DeltaMixer):
            mixer = PartSpec(
                kind="head_delta",
                args=dict(hidden_size=c.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
                          conv_taps=m.conv, eps=c.eps, gate_activation="silu"),
                tensors={"q_weight": Source.single(p + "q"), "k_weight": Source.single(p + "k"),
                         "v_weight": Source.single(p + "v"), "q_conv": Source.single(p + "q.conv"),
                         "k_conv": Source.single(p + "k.conv"), "v_conv": Source.single(p + "v.conv"),
                         "b_weight": Source.single(p + "b"), "a_weight": Source.single(p + "a"),
                         "g_weight": Source.single(p + "g"), "a_log": Source.single(p + "A_log"),
                         "dt_bias": Source.single(p + "dt_bias"), "out_norm": Source.single(p + "norm"),
                         "out_weight": Source.single(p + "o")})
        else:
            shares = m.kv_from is not None
            tensors = {"q_weight": Source.single(p + "q"), "uk_weight": Source.single(p + "uk"),
                       "uv_weight": Source.single(p + "uv"), "g_weight": Source.single(p + "g"),
                       "out_weight": Source.single(p + "o")}
            if shares:
                cache_of = m.kv_from          # schedule entry i runs layer i
            else:
                tensors.update({"dkv_weight": Source.single(p + "dkv"), "dkv_norm": Source.single(p + "dkv.norm")})
            mixer = PartSpec(
                kind="latent_attention",
                args=dict(hidden_size=c.width, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, kv_rank=m.kv_rank,
                          scale=m.scale, eps=c.eps, shares_latent=shares, gate_activation="sigmoid"),
                tensors=tensors)
        parts = {"mixer": mixer, "mixer_norm": norm(f"l{i}.norm1")}
        if layer.mlp is not None:
            parts.update({
                "ffn": PartSpec(kind="dense_act", args=dict(hidden_size=c.width, inner_size=layer.mlp.ff, activation="relu2"),
                                tensors={"up": Source.single(f"l{i}.mlp.up"), "down": Source.single(f"l{i}.mlp.down")}),
                "ffn_norm": norm(f"l{i}.norm2"),
            })
        layers.append(LayerSpec(block="outnorm", parts=parts))
        schedule.append(ScheduleEntry(layer=i, cache_of=cache_of))
    return ModelPlan(
        architecture=ARCHITECTURE,
        vocab_size=c.vocab,
        hidden_size=c.width,
        layers=layers,
        schedule=schedule,
        final_norm=norm("final.norm"),
        embedding=Source.single("embed"),
        lm_head=None,                   # the embedding table is the output matrix
        max_positions=MAX_POSITIONS,
        logit_softcap=c.logit_softcap,
        logit_scale=c.logit_scale,
    )


register_architecture(Architecture(
    name=ARCHITECTURE,
    config_from_json=config_from_json,
    plan=plan,
    config_to_json=config_to_json,
))
