"""Small Felepel configurations with sizes and constants of their own, and random weights for them."""
from __future__ import annotations

import json
import os

import numpy as np
import torch


def attention(heads, kv_heads, dim, vdim, scale=None, softcap=30.0, chunk=40):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale}
    if softcap is not None:
        m["softcap"] = softcap
    if chunk is not None:
        m["mask"] = {"size": chunk}
    return {"type": "attention", "mixer": m}


def delta(heads, kv_heads, dim, vdim, conv=4):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def moe(experts, top, ff, count=1, keep=1):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}


def config(width, vocab, layers, max_positions=512, eps=1e-5):
    """``layers``: (mixer entry, mlp or None) or ("of", j) for a layer that runs layer j's weights."""
    out = []
    for entry in layers:
        if entry[0] == "of":
            out.append({**{k: v for k, v in out[entry[1]].items() if k != "weights_of"}, "weights_of": entry[1]})
        else:
            out.append({**entry[0], "mlp": entry[1]})
    return {"architecture": "Felepel", "vocab": vocab, "width": width, "max_positions": max_positions,
            "norm": {"eps": eps}, "layers": out}


CASES = {
    # attention alone, delta rule alone, experts behind attention: each mechanism by itself
    "attention_only": config(64, 96, [(attention(4, 2, 16, 16, chunk=24), None)]),
    "delta_only": config(64, 96, [(delta(4, 4, 16, 16), None)]),
    "experts": config(48, 80, [(attention(2, 1, 16, 16, chunk=None, softcap=None), moe(8, 2, 24, 4, 2))]),
    # sizes that are no multiples of 16, 8 or 4; value width other than key width; fewer q/k heads than heads in the
    # delta rule; a chunk smaller than a page and one that is no divisor or multiple of it; 3 taps; a looped layer first
    "odd": config(72, 101, [
        (delta(6, 2, 20, 12, conv=3), moe(6, 1, 20, 3, 1)),
        (attention(6, 3, 20, 28, chunk=100, softcap=12.0), None),
        ("of", 0),
        (attention(3, 3, 24, 8, chunk=17, softcap=None, scale=0.31), moe(5, 5, 36)),
        ("of", 1),
    ]),
    # a width that is no multiple of four, two taps, five and one (no convolution at all), one expert of one, the attention first
    "ragged": config(50, 67, [
        (attention(5, 5, 10, 10, chunk=64), moe(1, 1, 10)),
        (delta(2, 1, 40, 24, conv=2), moe(9, 2, 18, 3, 2)),
        (delta(3, 3, 8, 70, conv=5), None),
        (delta(2, 2, 16, 8, conv=1), None),
    ]),
    # heads as wide as served models have them, and wider: key widths of 128, 192 and 256 (8 and 16 lanes to a value
    # channel in the recurrence's kernel, the last with rows to spare), value widths beyond one block of lanes
    "wide": config(256, 300, [
        (delta(4, 2, 128, 128), moe(8, 2, 128, 4, 2)),
        (attention(4, 1, 128, 128, chunk=64, softcap=50.0), None),
        (delta(1, 1, 256, 40, conv=2), None),
        (delta(2, 1, 192, 272, conv=3), None),
    ]),
    # as a served model's layers might be laid out, small: heads of 64, one kv head, groups, looped layers
    "regular": config(128, 256, [
        (delta(4, 4, 32, 32), moe(8, 2, 64, 2, 1)),
        (attention(4, 1, 64, 64, chunk=128, softcap=50.0), moe(8, 2, 64, 2, 1)),
        ("of", 0), ("of", 1),
    ], max_positions=1024),
}


def random_case(seed: int) -> tuple[dict, tuple[int, int]]:
    """A configuration drawn from sizes of many kinds (and the ranks of the delta rule's low-rank products, which only
    the tensors' shapes carry)."""
    rng = np.random.default_rng(7000 + seed)
    pick = lambda xs: xs[int(rng.integers(len(xs)))]
    divisors = lambda n: [d for d in range(1, n + 1) if n % d == 0]
    width = pick([40, 56, 64, 90, 96, 120, 160, 200, 256, 320])

    def mlp():
        if rng.random() < 0.25:
            return None
        experts = pick([2, 4, 6, 8, 12, 16])
        count = pick(divisors(experts))
        keep = int(rng.integers(1, count + 1))
        top = int(rng.integers(1, min(keep * (experts // count), 4) + 1))
        return moe(experts, top, pick([8, 20, 24, 40, 64, 100]), count, keep)

    layers = []
    for i in range(int(rng.integers(2, 6))):
        if i >= 1 and rng.random() < 0.3:
            own = [j for j, l in enumerate(layers) if l[0] != "of"]
            layers.append(("of", pick(own)))
            continue
        heads = pick([1, 2, 3, 4, 6, 8])
        kv = pick(divisors(heads))
        if rng.random() < 0.5:
            dim = pick([4, 8, 12, 16, 24, 32, 40, 48, 64, 80, 96])
            layers.append((attention(heads, kv, dim, pick([4, 8, 16, 24, 32, 48, 64, 72, 96]), scale=float(rng.uniform(0.5, 1.5)) * dim ** -0.5,
                                     softcap=pick([None, 20.0, 50.0]), chunk=pick([None, 7, 32, 50, 64, 96, 130])), mlp()))
        else:
            layers.append((delta(heads, kv, pick([4, 8, 16, 20, 32, 48, 64]), pick([4, 8, 16, 24, 32, 64, 96]),
                                 conv=pick([1, 2, 3, 4, 6])), mlp()))
    return config(width, int(rng.integers(50, 500)), layers, max_positions=256), (pick([3, 8, 24]), pick([5, 16]))


def tensors(cfg: dict, seed: int, peaky: float = 1.0, memory: float = 0.0, ranks: tuple[int, int] = (6, 10)) -> dict[str, np.ndarray]:
    """Random weights as float64 arrays whose values are bfloat16 numbers.  ``peaky`` scales the attention's query
    matrices, so that single keys decide a row of the softmax; ``memory`` is taken off A_log, so that the delta rule's
    state decays slowly and far tokens matter."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    out = {}

    def put(name, shape, std=1.0, mean=0.0):
        v = torch.tensor(rng.normal(mean, std, size=shape), dtype=torch.float32).to(torch.bfloat16)
        out[name] = v.to(torch.float64).numpy()

    put("embed", (cfg["vocab"], W))
    put("pos", (cfg["max_positions"], W), 0.5)
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", layer["mixer"]
        names = ["norm1", "norm1b"] + (["norm2", "norm2b"] if layer["mlp"] is not None else [])
        for n in names:
            put(p + n, (W,), 0.1, 1.0)
        H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        if layer["type"] == "attention":
            put(p + "mix.q", (H * D, W), peaky * W ** -0.5)
            put(p + "mix.k", (G * D, W), W ** -0.5)
            put(p + "mix.v", (G * V, W), W ** -0.5)
            for n, rows in (("q", H * D), ("k", G * D), ("v", G * V)):
                put(f"{p}mix.{n}.b", (rows,), 0.2)
            out[p + "mix.r1"] = torch.tensor(rng.uniform(0.0, 0.6, H), dtype=torch.float32).to(torch.bfloat16).double().numpy()
            out[p + "mix.r2"] = torch.tensor(rng.uniform(0.05, 2.0, H), dtype=torch.float32).to(torch.bfloat16).double().numpy()
            put(p + "mix.o", (W, H * V), (H * V) ** -0.5)
            put(p + "mix.o.b", (W,), 0.1)
        else:
            ra, rg = ranks
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * V)):
                put(f"{p}mix.{n}", (rows, W), W ** -0.5)
                put(f"{p}mix.{n}.conv", (rows, m["conv"]), 0.6)
            put(p + "mix.b", (H, W), W ** -0.5)
            put(p + "mix.A_log", (H,), 0.5, -memory)
            put(p + "mix.norm", (V,), 0.1, 1.0)
            put(p + "mix.a1", (ra, W), W ** -0.5)
            put(p + "mix.a2", (H * D, ra), ra ** -0.5)
            put(p + "mix.dt_bias", (H * D,), 1.0)
            put(p + "mix.g1", (rg, W), W ** -0.5)
            put(p + "mix.g2", (H * V, rg), rg ** -0.5)
            put(p + "mix.o", (W, H * V), (H * V) ** -0.5)
        f = layer["mlp"]
        if f is not None:
            ff = f["expert"]["ff"]
            for e in range(f["router"]["experts"]):
                put(f"{p}mlp.e{e}.gate", (ff, W), W ** -0.5)
                put(f"{p}mlp.e{e}.up", (ff, W), W ** -0.5)
                put(f"{p}mlp.e{e}.down", (W, ff), ff ** -0.5)
            put(p + "mlp.router", (f["router"]["experts"], W), 2.0 * W ** -0.5)
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
