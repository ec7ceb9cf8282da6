"""The Taminex design in the engine against the plain implementation in ``plain_taminex.py``: every mechanism alone, whole
prompts, decoding through the cache and the state, prompts in portions, unequal batches, slots and pages that are used
again, keys far away and at the borders of pages, sinks that take most of a row, latents shared between layers, long
decoding, sizes of many kinds, the kernels one by one, greedy generation through the library's entry point, and the
trace runner as a program."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch

import plain_taminex as plain
from taminex_cases import CASES, attention, config, dense, latent, random_case, tensors, tokens, write_folder

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_BOUND = 1e-4        # of the logits' root mean square, per position, mean taken off


@pytest.fixture(scope="module")
def made(tmp_path_factory):
    """(case, seed, peaky, memory, sink) -> (folder, config, weights), each written once."""
    cache = {}

    def get(case: str, seed: int = 0, peaky: float = 1.0, memory: float = 0.0, sink: float = 0.0):
        key = (case, seed, peaky, memory, sink)
        if key not in cache:
            cfg = CASES[case]
            w = tensors(cfg, seed, peaky, memory, sink)
            d = write_folder(str(tmp_path_factory.mktemp(f"taminex_{case}")), cfg, w)
            cache[key] = (d, cfg, w)
        return cache[key]
    return get


def engine_of(folder: str, dtype: str = "float32", max_tokens: int = 4096, **kw):
    from turboquant_cpp_amd.engine.model import load_model
    from turboquant_cpp_amd.engine.step import Engine
    return Engine(load_model(folder, act=dtype), max_tokens=max_tokens, page_size=64, **kw)


def errors(got, want: np.ndarray) -> np.ndarray:
    """Per position: root mean square of the difference with its mean taken off, over that of the wanted logits."""
    got = got.detach().double().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float64)
    d = got - want
    d = d - d.mean(axis=1, keepdims=True)
    scale = np.sqrt(np.mean((want - want.mean(axis=1, keepdims=True)) ** 2))
    return np.sqrt(np.mean(d * d, axis=1)) / scale


def check(got, want, dtype="float32", what=""):
    e = errors(got, want)
    if dtype == "float32":
        assert e.max() < F32_BOUND, f"{what}: position {int(e.argmax())} differs by {e.max():.2e}"
    elif dtype == "bfloat16":       # rounding of bfloat16 products and activations through all layers; a model of a few
        # dozen channels has positions where a norm divides by little and the rounding shows several times over
        assert e.max() < 0.2 and np.quantile(e, 0.9) < 0.06 and np.median(e) < 0.03, \
            f"{what}: median {np.median(e):.3f}, 90 % {np.quantile(e, 0.9):.3f}, worst {e.max():.3f} at {int(e.argmax())}"
    else:       # "same path": the engine against itself on another schedule, in bfloat16.  Where a head of the delta rule
        # reads next to nothing out of its state, its norm multiplies the rounding many times over (in 32 bits the same
        # positions stand out, at 1e-4): a few positions may differ by much, a fault of cache or state would change all
        assert np.quantile(e, 0.9) < 0.02 and e.max() < 0.5, \
            f"{what}: 90 % {np.quantile(e, 0.9):.3f}, position {int(e.argmax())} differs by {e.max():.2e}"


def wanted(eng, cfg, w, toks, dtype):
    """What a schedule's logits are held against, and how: in float32 the plain implementation; in bfloat16 the engine's
    own logits for the whole sequence in one step, alone (which test_whole_prompt_bfloat16 holds against the plain
    implementation): a schedule must not change them beyond rounding."""
    if dtype == "float32":
        return plain.forward(cfg, w, toks), dtype
    slot = eng.open(1)
    out = eng.step(slot, [toks], [all_places(len(toks))]).double().cpu().numpy()
    eng.close(slot)
    return out, "same path"


def all_places(n):
    return list(range(n))


def prompt_then_decode(eng, toks, cut):
    slot = eng.open(1)
    rows = [eng.step(slot, [toks[:cut]], [all_places(cut)])] + [eng.step(slot, [[t]]) for t in toks[cut:]]
    eng.close(slot)
    return torch.cat(rows)


# ---------------------------------------------------------------- whole prompts, every configuration
@pytest.mark.parametrize("case", sorted(CASES))
def test_whole_prompt(made, case):
    d, cfg, w = made(case)
    eng = engine_of(d)
    for seed, n in ((1, 1), (2, 150), (3, 67), (4, 2)):
        toks = tokens(cfg, n, seed)
        slot = eng.open(1)
        got = eng.step(slot, [toks], [all_places(n)])
        eng.close(slot)
        check(got, plain.forward(cfg, w, toks), what=f"{case}, {n} tokens")


@pytest.mark.parametrize("case", ["regular", "odd", "ragged", "wide", "widest"])
def test_whole_prompt_bfloat16(made, case):
    d, cfg, w = made(case)
    eng = engine_of(d, "bfloat16")
    toks = tokens(cfg, 200, 4)
    slot = eng.open(1)
    got = eng.step(slot, [toks], [all_places(len(toks))])
    check(got, plain.forward(cfg, w, toks), "bfloat16", case)


@pytest.mark.parametrize("seed", range(10))
def test_sizes_of_many_kinds(tmp_path, seed):
    """Configurations drawn at random: a prompt in two portions and a few decoded tokens, two requests side by side, in
    true 32-bit against the plain implementation at every position, and in bfloat16."""
    cfg = random_case(seed)
    w = tensors(cfg, seed)
    d = write_folder(str(tmp_path), cfg, w)
    a, b = tokens(cfg, 140, seed), tokens(cfg, 31, 100 + seed)
    wa, wb = plain.forward(cfg, w, a), plain.forward(cfg, w, b)
    for dtype in ("float32", "bfloat16"):
        eng = engine_of(d, dtype)
        sa, sb = eng.open(2)
        out = eng.step([sa, sb], [a[:70], b[:3]], [all_places(70), all_places(3)])
        rows_a, rows_b = [out[:70]], [out[70:]]
        out = eng.step([sa, sb], [a[70:130], b[3:]], [all_places(60), all_places(len(b) - 3)])
        rows_a.append(out[:60])
        rows_b.append(out[60:])
        eng.close([sb])
        rows_a += [eng.step([sa], [[t]]) for t in a[130:]]
        ga, gb = torch.cat(rows_a), torch.cat(rows_b)
        assert bool(torch.isfinite(ga).all()) and bool(torch.isfinite(gb).all())
        if dtype == "float32":
            check(ga, wa, what=f"seed {seed}: {json.dumps(cfg['layers'])}")
            check(gb, wb, what=f"seed {seed}, second request")
        else:
            assert np.median(errors(ga, wa)) < 0.05, f"seed {seed}: median {np.median(errors(ga, wa)):.3f}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_of_a_thousand_tokens(made, dtype):
    """Long enough for the plain products of the bfloat16 path to go to the vendor's library, over many pages, then
    decoded on."""
    d, cfg, w = made("regular", seed=7)
    eng = engine_of(d, dtype)
    toks = tokens(cfg, 1010, 13)
    check(prompt_then_decode(eng, toks, 1000), plain.forward(cfg, w, toks), dtype, "1,000 tokens")


def test_layers_one_by_one(made):
    """The residual stream behind every layer, layers on another's latents included."""
    d, cfg, w = made("odd")
    eng = engine_of(d)
    seen = []
    eng.layer_hook = lambda entry, hidden, batch: seen.append(hidden.double().cpu().numpy())
    toks = tokens(cfg, 45, 5)
    eng.step(eng.open(1), [toks], [[]])
    _, streams = plain.forward(cfg, w, toks, return_layers=True)
    assert len(seen) == len(cfg["layers"])
    for i, (a, b) in enumerate(zip(seen, streams)):
        assert np.abs(a - b).max() < 2e-4 * max(1.0, np.abs(b).max()), f"layer {i}"


# ---------------------------------------------------------------- decoding, portions, batches
@pytest.mark.parametrize("case,dtype", [("odd", "float32"), ("ragged", "float32"), ("regular", "float32"),
                                        ("regular", "bfloat16"), ("odd", "bfloat16"), ("ragged", "bfloat16"),
                                        ("wide", "float32"), ("wide", "bfloat16"), ("widest", "bfloat16"), ("shared_latent", "float32"),
                                        ("attention_only", "float32"), ("delta_only", "float32"), ("latent_only", "float32")])
def test_prompt_then_token_by_token(made, case, dtype):
    """Most of a sequence in one step, the rest one token a step (the later steps replayed as graphs), across the
    edges of pages."""
    d, cfg, w = made(case)
    eng = engine_of(d, dtype)
    toks = tokens(cfg, 150, 6)
    want, how = wanted(eng, cfg, w, toks, dtype)
    check(prompt_then_decode(eng, toks, 58), want, how, case)


def test_token_by_token_from_the_first(made):
    """No prompt step at all: the first tokens of a sequence through the decode kernels, an empty state, a convolution
    with nothing before it, a softmax over one key and the sink."""
    for case in ("odd", "ragged"):
        d, cfg, w = made(case, sink=2.0)
        eng = engine_of(d)
        toks = tokens(cfg, 70, 16)
        check(prompt_then_decode(eng, toks, 1), plain.forward(cfg, w, toks), what=case)


@pytest.mark.parametrize("case", ["odd", "ragged", "regular"])
def test_portions(made, case):
    """The logits do not depend on how a prompt was cut: portions of two tokens and more, of one, of a page and over."""
    d, cfg, w = made(case)
    eng = engine_of(d)
    toks = tokens(cfg, 190, 7)
    want = plain.forward(cfg, w, toks)
    for cuts in ([2, 3, 1, 5, 2, 64, 7, 2, 33, 71], [17, 2, 2, 100, 69], [95, 95], [64, 64, 62]):
        assert sum(cuts) == len(toks)
        slot, rows, at = eng.open(1), [], 0
        for c in cuts:
            rows.append(eng.step(slot, [toks[at:at + c]], [all_places(c)]))
            at += c
        eng.close(slot)
        check(torch.cat(rows), want, what=f"{case}, cuts {cuts}")


def test_portions_bfloat16(made):
    d, cfg, w = made("regular")
    eng = engine_of(d, "bfloat16")
    toks = tokens(cfg, 190, 7)
    want, how = wanted(eng, cfg, w, toks, "bfloat16")
    slot, rows, at = eng.open(1), [], 0
    for c in [2, 3, 1, 5, 2, 64, 7, 2, 33, 71]:
        rows.append(eng.step(slot, [toks[at:at + c]], [all_places(c)]))
        at += c
    check(torch.cat(rows), want, how, "portions")


@pytest.mark.parametrize("case,dtype", [("odd", "float32"), ("regular", "float32"), ("regular", "bfloat16"),
                                        ("ragged", "float32"), ("wide", "bfloat16"), ("widest", "bfloat16")])
def test_unequal_batch(made, case, dtype):
    """Requests of unequal lengths in one step and decoded together, the shorter ones ending earlier, against each
    alone in the plain implementation."""
    d, cfg, w = made(case)
    eng = engine_of(d, dtype)
    lengths, prompts = [1, 37, 131, 64, 90], [1, 20, 100, 64, 61]
    seqs = [tokens(cfg, n, 10 + i) for i, n in enumerate(lengths)]
    alone = [wanted(eng, cfg, w, s, dtype) for s in seqs]
    slots = eng.open(len(seqs))
    got = [[] for _ in seqs]
    out = eng.step(slots, [s[:p] for s, p in zip(seqs, prompts)], [all_places(p) for p in prompts])
    at = 0
    for i, p in enumerate(prompts):
        got[i].append(out[at:at + p])
        at += p
    done = list(prompts)
    while True:
        live = [i for i, s in enumerate(seqs) if done[i] < len(s)]
        if not live:
            break
        out = eng.step([slots[i] for i in live], [[seqs[i][done[i]]] for i in live])
        for r, i in enumerate(live):
            got[i].append(out[r:r + 1])
            done[i] += 1
            if done[i] == len(seqs[i]):
                eng.close([slots[i]])
    eng.close([slots[0]])
    for i, s in enumerate(seqs):
        check(torch.cat(got[i]), alone[i][0], alone[i][1], f"{case}, request {i}")


def test_slots_and_pages_used_again(made):
    """A cache with room for little: sequences come and go, each finds the pages and the slot of one before it, with
    that one's keys and latents in the pages and its state in the slot's row."""
    d, cfg, w = made("odd")
    eng = engine_of(d, max_tokens=256, max_slots=2)
    for round_ in range(3):
        a, b = tokens(cfg, 120 + round_, 20 + round_), tokens(cfg, 70, 30 + round_)
        sa, sb = eng.open(2)
        out = eng.step([sa, sb], [a[:100], b[:5]], [all_places(100), all_places(5)])
        rows_a, rows_b = [out[:100]], [out[100:]]
        eng.close([sa])
        rows_b.append(eng.step([sb], [b[5:]], [all_places(len(b) - 5)]))
        sc = eng.open(1)[0]
        assert sc == sa
        c = tokens(cfg, 66, 40 + round_)
        rows_c = [eng.step([sc], [c[:60]], [all_places(60)])] + [eng.step([sc], [[t]]) for t in c[60:]]
        eng.close([sb, sc])
        check(torch.cat(rows_a), plain.forward(cfg, w, a)[:100], what="first")
        check(torch.cat(rows_b), plain.forward(cfg, w, b), what="second")
        check(torch.cat(rows_c), plain.forward(cfg, w, c), what="in the first one's slot")
    assert all(v == 0 for v in eng.cache.pages_held().values())


# ---------------------------------------------------------------- far keys, borders of pages, sinks
def planted_attention(seed: int, sink: float):
    """One attention layer whose every query looks along the last channel of a head (which no rotation touches), where
    only token 1 has a key: wherever that token stands, it decides the rows behind it, against the sink."""
    D = 16
    cfg = config(32, 40, [(attention(2, 1, D, 16, rot=8, scale=1.0), None)])
    w = tensors(cfg, seed)
    w["embed"][:, 0] = 0.0
    w["embed"][1, 0] = 4.0
    for head in range(2):
        w["l0.mix.q.b"][head * D + D - 1] = 50.0          # after the head's norm: nearly sqrt(D) along the last channel
    w["l0.mix.k"][D - 1, :] = 0.0
    w["l0.mix.k"][D - 1, 0] = 50.0                          # token 1: a key of nearly sqrt(D) along it; all others: none
    w["l0.mix.k.b"][D - 1] = 0.0
    w["l0.mix.q.norm"][D - 1] = w["l0.mix.k.norm"][D - 1] = 1.0
    w["l0.mix.sink"][:] = sink
    return cfg, w


def planted_latent(seed: int):
    """One latent-attention layer: the first number of the latent is nonzero for token 1 only, every head's key along its
    first channel is that number, and every query looks along that channel."""
    D, R = 8, 24
    cfg = config(32, 40, [(latent(2, D, 16, R, scale=0.25), None)])
    w = tensors(cfg, seed)
    w["embed"][:, 0] = 0.0
    w["embed"][1, 0] = 4.0
    w["embed"][:, 1] = 2.0                                   # a channel that every token has
    w["l0.mix.dkv"][0, :] = 0.0
    w["l0.mix.dkv"][0, 0] = 8.0
    w["l0.mix.dkv.norm"][0] = 1.0
    for head in range(2):
        w["l0.mix.uk"][head * D, :] = 0.0
        w["l0.mix.uk"][head * D, 0] = 2.0
        w["l0.mix.q"][head * D, :] = 0.0
        w["l0.mix.q"][head * D, 1] = 3.0
    return cfg, w


@pytest.mark.parametrize("kind", ["attention", "latent"])
def test_a_key_far_back_and_at_the_borders_of_pages(tmp_path, kind):
    """The one token that every later query looks for stands at the first position, at a page's last and first places,
    or 300 tokens back; the rows behind it are read in a prompt and in decoding.  The plain implementation's own
    outputs with and without it differ by much, so a key that is lost or taken from a wrong place shows."""
    cfg, w = planted_attention(1, 0.0) if kind == "attention" else planted_latent(2)
    eng = engine_of(write_folder(str(tmp_path), cfg, w))
    n = 340
    base = [2 + (i * 7) % 38 for i in range(n)]
    without = plain.forward(cfg, w, base)
    for place in (0, 63, 64, 65, 127, 128, 255, 300):
        toks = list(base)
        toks[place] = 1
        want = plain.forward(cfg, w, toks)
        assert errors(want[place + 1:], without[place + 1:]).min() > 0.05, place
        for cut in (310, 62, 129):
            check(prompt_then_decode(eng, toks, cut), want, what=f"{kind}: the token at {place}, prompt of {cut}")


@pytest.mark.parametrize("sink", [-3.0, 4.0, 14.0])
def test_a_sink_against_one_strong_key(tmp_path, sink):
    """The planted key's score is about 16: a sink of 14 still takes a good part of every row behind it, and all of the
    rows before it, whose other scores are small; without the sink (or with it counted twice) the rows differ by much."""
    cfg, w = planted_attention(3, sink)
    eng = engine_of(write_folder(str(tmp_path), cfg, w))
    toks = [2 + (i * 5) % 38 for i in range(100)]
    toks[70] = 1
    want = plain.forward(cfg, w, toks)
    none = dict(w)
    none["l0.mix.sink"] = np.full(2, -1e9)
    if sink > 0:
        assert errors(plain.forward(cfg, none, toks), want).max() > 0.05
    check(prompt_then_decode(eng, toks, 66), want, what=f"sink {sink}")
    check(prompt_then_decode(eng, toks, 90), want, what=f"sink {sink}, key in the prompt")


def test_sinks_of_every_size_bfloat16(made):
    d, cfg, w = made("regular", seed=8, sink=3.0, peaky=3.0)
    eng = engine_of(d, "bfloat16")
    toks = tokens(cfg, 200, 4)
    check(prompt_then_decode(eng, toks, 180), plain.forward(cfg, w, toks), "bfloat16", "sinks")


def test_far_tokens_in_a_slowly_decaying_state(made):
    """Decays near 1: what the first tokens wrote into the state is still read hundreds of tokens later, in a prompt
    and in decoding; and queries that single keys decide."""
    d, cfg, w = made("odd", seed=3, peaky=6.0, memory=6.0)
    eng = engine_of(d)
    toks = tokens(cfg, 330, 9)
    want = plain.forward(cfg, w, toks)
    other = plain.forward(cfg, w, [(toks[0] + 1) % cfg["vocab"]] + toks[1:])
    assert errors(other[300:], want[300:]).max() > 50 * F32_BOUND      # the first token still matters at the end
    check(prompt_then_decode(eng, toks, 290), want, what="slow decay")
    check(prompt_then_decode(eng, toks, 5), want, what="slow decay, decoded")


def test_long_decoding(made):
    d, cfg, w = made("regular", seed=2)
    eng = engine_of(d)
    toks = tokens(cfg, 420, 11)
    check(prompt_then_decode(eng, toks, 3), plain.forward(cfg, w, toks), what="417 decoded tokens")


def test_values_that_a_model_may_happen_to_make_equal_or_one(tmp_path):
    """Scale 1 and other than dim^-1/2, logit scale 1 with a cap and a scale without one, one head, as many kv heads as
    heads, a value width other than the key width, a rotation base of 1 (every pair turns by the position itself)."""
    for i, cfg in enumerate([
        config(48, 60, [(attention(1, 1, 12, 20, rot=12, base=1.0, scale=1.0), dense(16)), (latent(1, 4, 12, 8, scale=1.0), None)],
               logit_scale=1.0, logit_softcap=5.0),
        config(48, 60, [(attention(3, 3, 16, 4, rot=2, scale=0.05), None), (latent(3, 16, 4, 33, scale=2.0), dense(48))],
               logit_scale=4.0),
    ]):
        w = tensors(cfg, 20 + i)
        eng = engine_of(write_folder(str(tmp_path / str(i)), cfg, w))
        toks = tokens(cfg, 90, 20 + i)
        check(prompt_then_decode(eng, toks, 70), plain.forward(cfg, w, toks), what=f"configuration {i}")


# ---------------------------------------------------------------- the mechanisms' kernels, one by one
def test_sum_of_a_normed_part_and_the_stream_itself():
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(0)
    for act in ("float32", "bfloat16"):
        for H, T, S in ((50, 7, 1), (72, 5, 3), (2048, 3, 2)):
            x, delta = rng.normal(size=(T, H)), rng.normal(size=(S, T, H))
            wd = rng.normal(1, 0.1, H)
            xg = torch.tensor(x, dtype=torch.float32, device="cuda")
            nd = ops.NormedDelta(torch.tensor(delta, dtype=torch.float32, device="cuda"),
                                 torch.tensor(wd, dtype=torch.float32, device="cuda"), 1e-5)
            h, _ = ops.add_rmsnorm(xg, nd, None, 0.0, act, stream=True)
            v = x + plain.rms_norm(delta.sum(0), wd, 1e-5)
            assert np.abs(xg.double().cpu().numpy() - v).max() < 1e-5           # the stream stays in 32 bits
            assert h.dtype == (torch.float32 if act == "float32" else torch.bfloat16)
            assert np.abs(h.double().cpu().numpy() - v).max() < (1e-5 if act == "float32" else 0.04)


def test_products_per_head_with_a_gate_and_the_latent_s_norm():
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(1)
    f32 = lambda a: torch.tensor(np.ascontiguousarray(a), dtype=torch.float32, device="cuda")
    for T, H, N, K in ((1, 3, 20, 12), (37, 2, 48, 32), (130, 5, 16, 304), (300, 4, 128, 64), (1, 4, 128, 512), (8, 3, 520, 128),
                       (16, 2, 24, 40), (5, 2, 16, 264)):
        a, wt, g = rng.normal(size=(T, H * K)), rng.normal(size=(H, N, K)), rng.normal(size=(T, H * N))
        want = np.einsum("thk,hnk->thn", a.reshape(T, H, K), wt).reshape(T, H * N)
        wide = f32(np.concatenate([rng.normal(size=(T, 5)), a, rng.normal(size=(T, 3))], axis=1))     # a run of columns
        got = ops.head_gemm(wide[:, 5:5 + H * K], f32(wt), "float32")
        assert np.abs(got.double().cpu().numpy() - want).max() < 1e-4 * np.abs(want).max()
        for name, f in (("sigmoid", plain.sigmoid), ("silu", plain.silu)):
            got = ops.head_gemm(f32(a), f32(wt), "float32", out_act=True, gate=f32(g), activation=name)
            assert np.abs(got.double().cpu().numpy() - want * f(g)).max() < 1e-4 * np.abs(want).max()
        got = ops.head_gemm(f32(a).bfloat16(), f32(wt).bfloat16(), "bfloat16", out_act=True, gate=f32(g), activation="sigmoid")
        assert got.dtype == torch.bfloat16
        assert np.abs(got.double().cpu().numpy() - want * plain.sigmoid(g)).max() < 0.03 * np.abs(want).max()
    for T, R, width, copies in ((1, 20, 32, 2), (70, 80, 80, 2), (9, 304, 304, 1), (33, 18, 32, 3)):
        src, wt = rng.normal(size=(T, R + 7)), rng.normal(1, 0.1, R)
        out = torch.full((T, copies * width + 2), 7.0, dtype=torch.float32, device="cuda")
        ops.latent_norm(f32(src)[:, 3:3 + R], f32(wt), 1e-5, out[:, 1:1 + copies * width], copies, width, "float32")
        got = out.double().cpu().numpy()
        want = plain.rms_norm(src[:, 3:3 + R], wt, 1e-5)
        assert np.all(got[:, 0] == 7.0) and np.all(got[:, -1] == 7.0)
        for c in range(copies):
            assert np.abs(got[:, 1 + c * width:1 + c * width + R] - want).max() < 1e-5
            assert np.all(got[:, 1 + c * width + R:1 + (c + 1) * width] == 0.0)


def test_activation_rows_and_scaled_capped_logits():
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(2)
    z = rng.normal(size=(9, 70)) * 3
    zg = torch.tensor(z, dtype=torch.float32, device="cuda")
    got = ops.act_rows(zg, None, "relu2", "float32")
    assert np.abs(got.double().cpu().numpy() - np.maximum(z, 0.0) ** 2).max() < 1e-5
    for scale, cap in ((2.5, 20.0), (0.5, None), (1.0, 4.0), (3.0, 1.5)):
        t = zg.clone()
        ops.softcap(t, cap, "float32", scale=scale)
        want = z * scale if cap is None else cap * np.tanh(z * scale / cap)
        assert np.abs(t.double().cpu().numpy() - want).max() < 1e-5


def test_a_product_whose_result_passes_an_activation():
    """In the product's own epilogue (few rows, tiles) and behind the vendor's product (many rows), in both types."""
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(3)
    for M, N, K in ((1, 96, 64), (8, 200, 128), (40, 136, 72), (300, 256, 264), (800, 128, 128)):
        a = torch.tensor(rng.normal(size=(M, K)), dtype=torch.float32, device="cuda")
        w = torch.tensor(rng.normal(size=(N, K)) * K ** -0.5, dtype=torch.float32, device="cuda")
        bias = torch.tensor(rng.normal(size=(N,)), dtype=torch.float32, device="cuda")
        for act, dt, tol in (("float32", torch.float32, 1e-4), ("bfloat16", torch.bfloat16, 0.04)):
            aa, ww = a.to(dt), w.to(dt)
            z = aa.double().cpu().numpy() @ ww.double().cpu().numpy().T
            for name, f in (("relu2", lambda v: np.maximum(v, 0.0) ** 2), ("silu", plain.silu)):
                got = ops.gemm(aa, ww, act, activation=name, act_alone=True)
                assert got.dtype == dt and np.abs(got.double().cpu().numpy() - f(z)).max() < tol * max(1.0, np.abs(f(z)).max())
            got = ops.gemm(aa, ww, act, bias=bias, activation="relu2", act_alone=True)
            want = np.maximum(z + bias.double().cpu().numpy(), 0.0) ** 2
            assert np.abs(got.double().cpu().numpy() - want).max() < tol * max(1.0, np.abs(want).max())
            plain_product = ops.gemm(aa, ww, act)          # and nothing of it sticks to the next plain product
            assert np.abs(plain_product.double().cpu().numpy() - z).max() < tol * max(1.0, np.abs(z).max())


def test_delta_rule_kernels_with_a_state_carried_over(made):
    """The mixer's kernels against the plain function, the sequence cut in three runs so that each starts from the one
    before's state and convolution inputs, the last through the decode step's single kernel; two sequences side by side
    in slots far apart."""
    from turboquant_cpp_amd.csrc import ops
    for case, layer in (("ragged", 1), ("ragged", 2), ("odd", 0), ("ragged", 4), ("wide", 0)):
        _, cfg, w = made(case)
        m, p = cfg["layers"][layer]["mixer"], f"l{layer}.mix."
        H, G, D, V, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        dims = ops.DeltaDims(H, G, D, V, K, 0, 0, head_decay=True)
        rng = np.random.default_rng(layer)
        lens, slots = (23, 1), (5, 2)
        hs = [rng.normal(size=(n + 10, cfg["width"])) for n in lens]
        want = [plain.head_delta(h, m, w, p, 1e-5, return_state=True) for h in hs]
        dev = "cuda"
        f32 = lambda a: torch.tensor(np.ascontiguousarray(a), dtype=torch.float32, device=dev)
        state = torch.zeros((8, dims.state_floats + 3), dtype=torch.float32, device=dev)
        w_in = np.concatenate([w[p + n] for n in ("q", "k", "v", "b", "a", "g")])
        conv = f32(np.concatenate([w[p + n] for n in ("q.conv", "k.conv", "v.conv")]))
        a_log, dt_bias, norm_w = f32(w[p + "A_log"]), f32(w[p + "dt_bias"]), f32(w[p + "norm"])
        outs = [[], []]
        for run in range(3):
            parts = [h[:n] if run == 0 else h[n:n + 9] if run == 1 else h[n + 9:] for h, n in zip(hs, lens)]
            x = np.concatenate(parts)
            cu = np.cumsum([0] + [len(q) for q in parts])
            runs = {"cu_seqlens": torch.tensor(cu, dtype=torch.int32, device=dev),
                    "slots": torch.tensor(slots, dtype=torch.int32, device=dev), "decode": run == 2}
            slot_of_token = torch.tensor(np.repeat(slots, [len(q) for q in parts]), dtype=torch.int32, device=dev)
            proj = f32(x @ w_in.T)
            qn, kn, vc, beta, dec = ops.delta_prep_h(proj, slot_of_token, state, conv, a_log, dt_bias, dims, "float32")
            if run == 2 and ops.delta_decode_fits(dims):
                out = ops.delta_decode_h(qn, kn, vc, beta, a_log, dt_bias, norm_w, 1e-5, proj, "silu", runs, state, dims, "float32")
            else:
                o = ops.delta_scan_h(qn, kn, vc, beta, dec, runs, state, dims, "float32")
                out = ops.delta_out_h(o, norm_w, 1e-5, proj, "silu", runs, state, dims, "float32")
            y = out.double().cpu().numpy() @ w[p + "o"].T
            for i in range(2):
                outs[i].append(y[cu[i]:cu[i + 1]])
        for i in range(2):
            got = np.concatenate(outs[i])
            assert np.abs(got - want[i][0]).max() < 2e-5 * max(1.0, np.abs(want[i][0]).max()), (case, layer, i)
            S = state[slots[i], :H * D * V].double().cpu().numpy().reshape(H, D, V)
            assert np.abs(S - want[i][1]).max() < 2e-5 * max(1.0, np.abs(want[i][1]).max())
        assert float(state[0].abs().max()) == 0.0 and float(state[:, dims.state_floats:].abs().max()) == 0.0


# ---------------------------------------------------------------- the library's own entry points
def test_greedy_generation_through_the_entry_point(made):
    from turboquant_cpp_amd import Model
    d, cfg, w = made("regular", seed=5)
    prompts = [tokens(cfg, n, 50 + n) for n in (5, 70, 1, 33)]
    with Model(d, dtype="float32", temperature=0.0, rep_penalty=1.0, max_tokens=24, max_batch=3, stop_tokens=()) as m:
        got = m.generate(prompts, loop_detection=False)
    for p, g in zip(prompts, got):
        assert len(g) == 24
        rows = plain.forward(cfg, w, p + g)
        for j, tok in enumerate(g):
            row = rows[len(p) - 1 + j]
            assert row[tok] >= row.max() - 1e-3, f"token {j} of a prompt of {len(p)} is not the plain model's choice"


def test_a_conversation_over_state_and_shared_latents(made, tmp_path):
    """``Model.chat``: a turn that goes on runs only the new tokens; a history that parts from the cached tokens starts
    over (a state has no earlier value); a saved conversation goes on in another model object with the same tokens."""
    from turboquant_cpp_amd import Model
    d, cfg, w = made("regular", seed=5)
    opts = dict(dtype="float32", temperature=0.0, rep_penalty=1.0, max_tokens=5, context_length=512)
    h1, extra, other, more = (tokens(cfg, n, 70 + n) for n in (70, 9, 150, 5))
    with Model(d, **opts) as m, Model(d, **opts) as fresh:
        brought = []
        step = m.engine.step
        m.engine.step = lambda slots, toks, *a, **k: (brought.append(len(toks[0])), step(slots, toks, *a, **k))[1]
        out1 = m.chat(h1)
        assert out1 == fresh.generate([h1])[0] and brought[0] == 70
        del brought[:]
        h2 = h1 + out1 + extra
        out2 = m.chat(h2)
        assert brought[0] == 1 + len(extra) and out2 == fresh.generate([h2])[0]
        saved = str(tmp_path / "talk.kv")
        m.save_context(saved)
        del brought[:]
        h3 = h1[:40] + other
        assert m.chat(h3) == fresh.generate([h3])[0] and brought[0] == len(h3)
        with Model(d, **opts) as later:
            later.load_context(saved)
            h4 = h2 + out2 + more
            assert later.chat(h4) == fresh.generate([h4])[0]


def test_command_line(made):
    """``bin/quant``: what it says of the folder, and greedy tokens that are the entry point's."""
    from turboquant_cpp_amd import Model
    d, cfg, w = made("regular", seed=5)
    quant = os.path.join(ROOT, "bin", "quant")
    info = subprocess.run([quant, d, "--info"], capture_output=True, text=True, timeout=300)
    assert info.returncode == 0 and "Taminex" in info.stdout, info.stderr[-1000:]
    run = subprocess.run([quant, d, "-p", "5,17,3;8,1", "-n", "6", "-T", "0", "--rep-penalty", "1.0", "--dtype", "float32",
                          "--json", "-M"], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    with Model(d, dtype="float32", temperature=0.0, rep_penalty=1.0, max_tokens=6) as m:
        want = m.generate([[5, 17, 3], [8, 1]])
    got = [r["tokens"] for r in json.loads(run.stdout.strip().splitlines()[-1])]
    assert got == want


def test_trace_runner_as_a_program(made, tmp_path):
    d, cfg, w = made("odd", seed=6)
    a, b = tokens(cfg, 90, 60), tokens(cfg, 41, 61)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:80], "want": [0, 41, 79]}, {"id": "b", "tokens": b[:40], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[80:81], "want": [0]}, {"id": "b", "tokens": b[40:], "want": [0]}], "end": ["b"]}]
    steps += [{"step": 2 + i, "entries": [{"id": "a", "tokens": [t], "want": [0] if i % 2 else []}], "end": ["a"] if i == 8 else []}
              for i, t in enumerate(a[81:])]
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / dtype
        run = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype, "--out", str(out),
                              "--max-tokens", "256"], input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                             capture_output=True, timeout=600)
        assert run.returncode == 0, run.stderr[-2000:]
        assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        wa, wb = plain.forward(cfg, w, a), plain.forward(cfg, w, b)
        V = cfg["vocab"]
        read = lambda i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V)
        check(read(0), wa[[0, 41, 79]], dtype, what="step 0")
        check(read(1), np.stack([wa[80], wb[40]]), dtype, what="step 1")
        for i in range(9):
            if i % 2:
                check(read(2 + i), wa[81 + i:82 + i], dtype, what=f"step {2 + i}")
            else:
                assert not (out / f"{2 + i}.f32").exists()
