"""Small Taminex configurations with sizes and constants of their own, and random weights for them."""
from __future__ import annotations

import json
import os

import numpy as np
import torch


def attention(heads, kv_heads, dim, vdim, scale=None, rot=None, base=10000.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale,
         "rot": {"dims": dim if rot is None else rot, "base": base}}
    return {"type": "attention", "mixer": m}


def delta(heads, kv_heads, dim, vdim, conv=4):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def latent(heads, dim, vdim, kv_rank, scale=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": dim ** -0.5 if scale is None else scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def config(width, vocab, layers, eps=1e-5, logit_scale=1.0, logit_softcap=None):
    """``layers``: (mixer entry, mlp or None)."""
    out = {"architecture": "Taminex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
           "layers": [{**mixer, "mlp": mlp} for mixer, mlp in layers]}
    if logit_softcap is not None:
        out["logit_softcap"] = logit_softcap
    return out


CASES = {
    # each mechanism by itself
    "attention_only": config(64, 96, [(attention(4, 2, 16, 16, rot=8), None)]),
    "delta_only": config(64, 96, [(delta(4, 2, 16, 16), None)]),
    "latent_only": config(64, 96, [(latent(4, 16, 16, 24), None)], logit_scale=1.5),
    "shared_latent": config(48, 80, [(latent(2, 8, 16, 20), dense(40)), (latent(3, 16, 8, 20, kv_from=0), None)], logit_softcap=10.0),
    "ff_only_behind_attention": config(40, 50, [(attention(1, 1, 8, 8), dense(24))], logit_scale=3.0, logit_softcap=8.0),
    # sizes that are no multiples of 16, 8 or 4; value width other than key width; as many kv heads as heads and one kv
    # head; rotation of a whole head, of a part, of nothing; 1, 2, 3 and 5 taps; a latent no multiple of 16; two layers
    # on one layer's latents, with another latent layer of its own between them; a delta layer first, attention last
    "odd": config(72, 101, [
        (delta(6, 2, 20, 12, conv=3), dense(36)),
        (latent(3, 12, 20, 40, scale=0.4), None),
        (attention(6, 3, 20, 28, rot=12, base=500.0, scale=0.31), dense(50)),
        (latent(5, 8, 8, 40, kv_from=1), dense(30)),
        (latent(2, 24, 12, 18), None),
        (latent(4, 20, 4, 40, kv_from=1, scale=0.2), None),
        (attention(3, 3, 24, 8, rot=0), None),
    ], logit_scale=0.7, logit_softcap=25.0),
    # a width that is no multiple of four, heads of 10, a convolution of one tap (none at all)
    "ragged": config(50, 67, [
        (attention(5, 5, 10, 10, rot=10, base=77.0), dense(10)),
        (delta(2, 1, 40, 24, conv=2), dense(18)),
        (delta(3, 3, 8, 70, conv=5), None),
        (latent(5, 10, 6, 50), dense(22)),
        (delta(2, 2, 16, 8, conv=1), None),
    ], eps=1e-6, logit_softcap=15.0),
    # heads as wide as served models have them: key widths of 128, 192 and 256 in the recurrence, heads of 128 in both
    # attentions, a latent of 256 and one beyond the matrix-core attention's widths
    "wide": config(256, 300, [
        (delta(4, 2, 128, 128), dense(512)),
        (attention(4, 1, 128, 128, rot=64, base=1e6), None),
        (latent(4, 128, 128, 256), dense(256)),
        (delta(1, 1, 256, 40, conv=2), None),
        (latent(2, 64, 64, 256, kv_from=2), None),
        (delta(2, 1, 192, 272, conv=3), None),
        (latent(2, 32, 48, 304), None),
    ], logit_scale=2.5, logit_softcap=40.0),
    # latents as wide as the attention kernels take them, and just below
    "widest": config(128, 200, [
        (latent(2, 32, 32, 512), dense(64)),
        (latent(4, 16, 16, 512, kv_from=0), None),
        (latent(2, 32, 16, 496), None),
    ], logit_softcap=20.0),
    # as a served model's layers might be laid out, small
    "regular": config(128, 256, [
        (delta(4, 2, 32, 48), dense(192)),
        (attention(4, 1, 64, 64, rot=16, base=1e5), dense(192)),
        (delta(4, 4, 32, 64), dense(320)),
        (latent(4, 32, 32, 64), dense(192)),
        (latent(4, 32, 32, 64, kv_from=3), dense(320)),
    ], logit_scale=1.5, logit_softcap=24.0),
}


def random_case(seed: int) -> dict:
    """A configuration drawn from sizes of many kinds."""
    rng = np.random.default_rng(9000 + seed)
    pick = lambda xs: xs[int(rng.integers(len(xs)))]
    divisors = lambda n: [d for d in range(1, n + 1) if n % d == 0]
    width = pick([40, 56, 64, 90, 96, 120, 160, 200, 256])
    layers = []
    for i in range(int(rng.integers(2, 7))):
        mlp = None if rng.random() < 0.3 else dense(pick([8, 20, 24, 40, 64, 100, 130]))
        heads = pick([1, 2, 3, 4, 6, 8])
        kind = rng.random()
        own = [j for j, (l, _) in enumerate(layers) if l["type"] == "latent_attention" and "kv_from" not in l["mixer"]]
        if kind < 0.3:
            dim = pick([4, 8, 12, 16, 24, 32, 40, 48, 64, 80, 96])
            layers.append((attention(heads, pick(divisors(heads)), dim, pick([4, 8, 16, 24, 32, 48, 64, 72, 96]),
                                     scale=float(rng.uniform(0.5, 1.5)) * dim ** -0.5, rot=pick([0, 2, dim // 2 // 2 * 2, dim]),
                                     base=pick([100.0, 1e4, 1e6])), mlp))
        elif kind < 0.6:
            layers.append((delta(heads, pick(divisors(heads)), pick([4, 8, 16, 20, 32, 48, 64]), pick([4, 8, 16, 24, 32, 64, 96]),
                                 conv=pick([1, 2, 3, 4, 6])), mlp))
        elif own and rng.random() < 0.5:
            src = pick(own)
            dim = pick([4, 8, 16, 24, 32, 64])
            layers.append((latent(heads, dim, pick([4, 8, 16, 24, 32, 64]), layers[src][0]["mixer"]["kv_rank"],
                                  scale=float(rng.uniform(0.5, 1.5)) * dim ** -0.5, kv_from=src), mlp))
        else:
            dim = pick([4, 8, 16, 24, 32, 64])
            layers.append((latent(heads, dim, pick([4, 8, 16, 24, 32, 64]), pick([8, 16, 20, 48, 64, 100, 128]),
                                  scale=float(rng.uniform(0.5, 1.5)) * dim ** -0.5), mlp))
    return config(width, int(rng.integers(50, 500)), layers, eps=pick([1e-5, 1e-6]), logit_scale=pick([1.0, 0.5, 2.0]),
                  logit_softcap=pick([None, 20.0, 50.0]))


def tensors(cfg: dict, seed: int, peaky: float = 1.0, memory: float = 0.0, sink: float = 0.0) -> dict[str, np.ndarray]:
    """Random weights as float64 arrays whose values are bfloat16 numbers.  ``peaky`` scales the attentions' query
    matrices, so that single keys decide a row of the softmax; ``memory`` is taken off A_log, so that the delta rule's
    state decays slowly and far tokens matter; ``sink`` is the mean of the sinks."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    out = {}

    def put(name, shape, std=1.0, mean=0.0):
        v = torch.tensor(rng.normal(mean, std, size=shape), dtype=torch.float32).to(torch.bfloat16)
        out[name] = v.to(torch.float64).numpy()

    put("embed", (cfg["vocab"], W))
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        put(p + "norm1", (W,), 0.1, 1.0)
        H, D, V = m["heads"], m["dim"], m["vdim"]
        if layer["type"] == "attention":
            G = m["kv_heads"]
            put(p + "mix.q", (H * D, W), peaky * W ** -0.5)
            put(p + "mix.k", (G * D, W), W ** -0.5)
            put(p + "mix.v", (G * V, W), W ** -0.5)
            for n, rows in (("q", H * D), ("k", G * D), ("v", G * V)):
                put(f"{p}mix.{n}.b", (rows,), 0.2)
            put(p + "mix.q.norm", (D,), 0.2, peaky)
            put(p + "mix.k.norm", (D,), 0.2, 1.0)
            put(p + "mix.sink", (H,), 1.0, sink)
            put(p + "mix.o", (W, H * V), (H * V) ** -0.5)
        elif layer["type"] == "delta":
            G = m["kv_heads"]
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * V)):
                put(f"{p}mix.{n}", (rows, W), W ** -0.5)
                put(f"{p}mix.{n}.conv", (rows, m["conv"]), 0.6)
            put(p + "mix.b", (H, W), W ** -0.5)
            put(p + "mix.a", (H, W), W ** -0.5)
            put(p + "mix.A_log", (H,), 0.5, -memory)
            put(p + "mix.dt_bias", (H,), 1.0)
            put(p + "mix.norm", (V,), 0.1, 1.0)
            put(p + "mix.g", (H * V, W), W ** -0.5)
            put(p + "mix.o", (W, H * V), (H * V) ** -0.5)
        else:
            R = m["kv_rank"]
            put(p + "mix.q", (H * D, W), peaky * W ** -0.5)
            if m.get("kv_from") is None:
                put(p + "mix.dkv", (R, W), W ** -0.5)
                put(p + "mix.dkv.norm", (R,), 0.1, 1.0)
            put(p + "mix.uk", (H * D, R), R ** -0.5)
            put(p + "mix.uv", (H * V, R), R ** -0.5)
            put(p + "mix.g", (H * V, W), W ** -0.5)
            put(p + "mix.o", (W, H * V), (H * V) ** -0.5)
        f = layer["mlp"]
        if f is not None:
            put(p + "norm2", (W,), 0.1, 1.0)
            put(p + "mlp.up", (f["ff"], W), W ** -0.5)
            put(p + "mlp.down", (W, f["ff"]), f["ff"] ** -0.5)
    put("final.norm", (W,), 0.1, 1.0)
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
