"""The Felepel design in the engine against the plain implementation in ``plain_felepel.py``: every mechanism alone,
whole prompts, decoding through the cache and the state, prompts in portions, unequal batches, slots and pages that
are used again, keys at the edges of chunks and far away, long decoding, sizes of many kinds, greedy generation
through the library's entry point, and the trace runner as a program."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_felepel as plain
from felepel_cases import CASES, random_case, tensors, tokens, write_folder

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_BOUND = 1e-4        # of the logits' root mean square, per position, mean taken off


@pytest.fixture(scope="module")
def made(tmp_path_factory):
    """(case, seed, peaky, memory) -> (folder, config, weights), each written once."""
    cache = {}

    def get(case: str, seed: int = 0, peaky: float = 1.0, memory: float = 0.0):
        key = (case, seed, peaky, memory)
        if key not in cache:
            cfg = CASES[case]
            w = tensors(cfg, seed, peaky, memory)
            d = write_folder(str(tmp_path_factory.mktemp(f"felepel_{case}")), cfg, w)
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
    elif dtype == "bfloat16":
        # rounding of bfloat16 products, and now and then an expert chosen otherwise behind it, which the delta rule's
        # state then carries along for some tokens: most positions are close, not all
        assert np.quantile(e, 0.75) < 0.06 and np.median(e) < 0.03, f"{what}: median {np.median(e):.3f}, 75 % {np.quantile(e, 0.75):.3f}"
    else:       # "same path": the engine against itself on another schedule, in bfloat16
        assert e.max() < 0.02, f"{what}: position {int(e.argmax())} differs by {e.max():.2e}"


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


# ---------------------------------------------------------------- whole prompts, every configuration
@pytest.mark.parametrize("case", sorted(CASES))
def test_whole_prompt(made, case):
    d, cfg, w = made(case)
    eng = engine_of(d)
    for seed, n in ((1, 1), (2, 150), (3, 67)):
        toks = tokens(cfg, n, seed)
        slot = eng.open(1)
        got = eng.step(slot, [toks], [all_places(n)])
        eng.close(slot)
        check(got, plain.forward(cfg, w, toks), what=f"{case}, {n} tokens")


@pytest.mark.parametrize("case", ["regular", "odd", "ragged", "wide"])
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
    true 32-bit against the plain implementation at every position, and in bfloat16, where most positions are close."""
    cfg, ranks = random_case(seed)
    w = tensors(cfg, seed, ranks=ranks)
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
            # (five layers of experts behind rounded activations: choices differ here and there, and stay differing)
            assert np.median(errors(ga, wa)) < 0.1, f"seed {seed}: median {np.median(errors(ga, wa)):.3f}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_of_a_thousand_tokens(made, dtype):
    """Long enough for the plain products of the bfloat16 path to go to the vendor's library, over many chunks and pages,
    then decoded on."""
    d, cfg, w = made("regular", seed=7)
    eng = engine_of(d, dtype)
    toks = tokens(cfg, 1010, 13)
    want = plain.forward(cfg, w, toks)
    slot = eng.open(1)
    rows = [eng.step(slot, [toks[:1000]], [all_places(1000)])] + [eng.step(slot, [[t]]) for t in toks[1000:]]
    check(torch.cat(rows), want, dtype, "1,000 tokens")


def test_layers_one_by_one(made):
    """The residual stream behind every layer run, looped layers included."""
    d, cfg, w = made("odd")
    eng = engine_of(d)
    seen = []
    eng.layer_hook = lambda entry, hidden, batch: seen.append(hidden.double().cpu().numpy())
    toks = tokens(cfg, 45, 5)
    eng.step(eng.open(1), [toks], [[]])
    _, streams = plain.forward(cfg, w, toks, return_layers=True)
    assert len(seen) == len(cfg["layers"])
    for i, (a, b) in enumerate(zip(seen, streams)):
        assert np.abs(a - b).max() < 2e-4 * max(1.0, np.abs(b).max()), f"layer run {i}"


# ---------------------------------------------------------------- decoding, portions, batches
@pytest.mark.parametrize("case,dtype", [("odd", "float32"), ("ragged", "float32"), ("regular", "float32"),
                                        ("regular", "bfloat16"), ("odd", "bfloat16"), ("ragged", "bfloat16"),
                                        ("wide", "float32"), ("wide", "bfloat16")])
def test_prompt_then_token_by_token(made, case, dtype):
    """Most of a sequence in one step, the rest one token a step (the later steps replayed as graphs), across the
    edges of chunks and pages."""
    d, cfg, w = made(case)
    eng = engine_of(d, dtype)
    toks = tokens(cfg, 150, 6)
    want, how = wanted(eng, cfg, w, toks, dtype)
    slot = eng.open(1)
    rows = [eng.step(slot, [toks[:58]], [all_places(58)])]
    for t in toks[58:]:
        rows.append(eng.step(slot, [[t]]))
    check(torch.cat(rows), want, how, case)


@pytest.mark.parametrize("case", ["odd", "ragged", "regular"])
def test_portions(made, case):
    """The logits do not depend on how a prompt was cut: portions of two tokens and more, of one, of a page and over."""
    d, cfg, w = made(case)
    eng = engine_of(d)
    toks = tokens(cfg, 190, 7)
    want = plain.forward(cfg, w, toks)
    for cuts in ([2, 3, 1, 5, 2, 64, 7, 2, 33, 71], [17, 2, 2, 100, 69], [95, 95]):
        assert sum(cuts) == len(toks)
        slot, rows, at = eng.open(1), [], 0
        for c in cuts:
            rows.append(eng.step(slot, [toks[at:at + c]], [all_places(c)]))
            at += c
        eng.close(slot)
        check(torch.cat(rows), want, what=f"{case}, cuts {cuts}")


@pytest.mark.parametrize("case,dtype", [("odd", "float32"), ("regular", "float32"), ("regular", "bfloat16")])
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
    that one's keys in the pages and its state in the slot's row."""
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
        rows_c = eng.step([sc], [c], [all_places(len(c))])
        eng.close([sb, sc])
        check(torch.cat(rows_a), plain.forward(cfg, w, a)[:100], what="first")
        check(torch.cat(rows_b), plain.forward(cfg, w, b), what="second")
        check(rows_c, plain.forward(cfg, w, c), what="in the first one's slot")
    assert all(v == 0 for v in eng.cache.pages_held().values())


def test_chunks_give_their_pages_back(made):
    d, cfg, w = made("attention_only")          # chunks of 24 positions, pages of 64
    eng = engine_of(d)
    slot = eng.open(1)
    toks = tokens(cfg, 300, 8)
    eng.step(slot, [toks[:200]], [[]])
    assert sum(eng.cache.pages_held().values()) == 1      # position 200 sees 192.., which lies in the page of 192..255
    rows = [eng.step(slot, [[t]]) for t in toks[200:]]
    assert sum(eng.cache.pages_held().values()) <= 2
    check(torch.cat(rows), plain.forward(cfg, w, toks)[200:], what="decoding after pages were given back")


# ---------------------------------------------------------------- edges of chunks, far keys
def planted_attention(chunk: int, seed: int):
    """One attention layer whose every query looks hard for the key of token 1: where that token lies just inside or
    just outside a query's chunk decides the output."""
    from felepel_cases import attention, config
    cfg = config(32, 40, [(attention(2, 1, 16, 16, chunk=chunk, softcap=40.0, scale=1.0), None)], max_positions=512)
    w = tensors(cfg, seed)
    w["pos"] *= 0.0
    k, q = w["l0.mix.k"], w["l0.mix.q"]
    k *= 0.05
    q *= 0.05
    w["l0.mix.k.b"][:] = 0.0
    w["l0.mix.q.b"][:] = 0.0
    w["l0.mix.q.b"][0] = w["l0.mix.q.b"][16] = 6.0       # every query: 6 along the first key channel, in both heads
    w["embed"][1] = 0.0
    w["embed"][1][0] = 4.0                                 # token 1 after the norm: (sqrt(32), 0, 0, ...)
    w["l0.norm1"][:] = 1.0
    k[0, :] = 0.0
    k[0, 0] = 1.0                                          # its key: 5.7 along that channel, a score of 34
    return cfg, w


@pytest.mark.parametrize("chunk", [16, 24, 64, 100])
def test_key_just_inside_and_just_outside_a_chunk(tmp_path, chunk):
    cfg, w = planted_attention(chunk, chunk)
    eng = engine_of(write_folder(str(tmp_path), cfg, w))
    n = 3 * chunk + 5
    outs = {}
    for where in ("inside", "outside"):
        for start in (chunk, 2 * chunk):              # the edge in a prompt, and the edge passed while decoding
            toks = [2 + (i * 7) % 38 for i in range(n)]
            toks[start if where == "inside" else start - 1] = 1
            want = plain.forward(cfg, w, toks)
            slot = eng.open(1)
            got = [eng.step(slot, [toks[:2 * chunk - 3]], [all_places(2 * chunk - 3)])]
            got += [eng.step(slot, [[t]]) for t in toks[2 * chunk - 3:]]
            eng.close(slot)
            check(torch.cat(got), want, what=f"chunk {chunk}, token {where} at {start}")
            outs[where, start] = want
    # the plain implementation itself tells the two places apart, by much: the test can see an edge that is one off
    for start in (chunk, 2 * chunk):
        rows = slice(start, start + chunk)
        assert np.abs(outs["inside", start][rows] - outs["outside", start][rows]).max() > 0.5


def test_far_tokens_in_a_slowly_decaying_state(made):
    """Decays near 1: what the first tokens wrote into the state is still read hundreds of tokens later, in a prompt
    and in decoding; and queries that single keys decide."""
    d, cfg, w = made("odd", seed=3, peaky=6.0, memory=6.0)
    eng = engine_of(d)
    toks = tokens(cfg, 330, 9)
    want = plain.forward(cfg, w, toks)
    other = plain.forward(cfg, w, [(toks[0] + 1) % cfg["vocab"]] + toks[1:])
    assert errors(other[300:], want[300:]).max() > 50 * F32_BOUND      # the first token still matters at the end
    slot = eng.open(1)
    rows = [eng.step(slot, [toks[:290]], [all_places(290)])] + [eng.step(slot, [[t]]) for t in toks[290:]]
    check(torch.cat(rows), want, what="slow decay")


def test_long_decoding(made):
    d, cfg, w = made("regular", seed=2)
    eng = engine_of(d)
    toks = tokens(cfg, 420, 11)
    slot = eng.open(1)
    rows = [eng.step(slot, [toks[:3]], [all_places(3)])] + [eng.step(slot, [[t]]) for t in toks[3:]]
    check(torch.cat(rows), plain.forward(cfg, w, toks), what="417 decoded tokens")


# ---------------------------------------------------------------- the mechanisms' kernels, one by one
def test_sum_of_a_normed_part_and_norm():
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(0)
    for H, T, S in ((50, 7, 1), (72, 5, 3), (2048, 3, 2)):
        x, delta = rng.normal(size=(T, H)), rng.normal(size=(S, T, H))
        wd, w = rng.normal(1, 0.1, H), rng.normal(1, 0.1, H)
        xg = torch.tensor(x, dtype=torch.float32, device="cuda")
        nd = ops.NormedDelta(torch.tensor(delta, dtype=torch.float32, device="cuda"),
                             torch.tensor(wd, dtype=torch.float32, device="cuda"), 1e-5)
        out, out32 = ops.add_rmsnorm(xg, nd, torch.tensor(w, dtype=torch.float32, device="cuda"), 1e-6, "float32", want_f32=True)
        v = x + plain.rms_norm(delta.sum(0), wd, 1e-5)
        assert np.abs(xg.double().cpu().numpy() - v).max() < 1e-5
        assert np.abs(out32.double().cpu().numpy() - plain.rms_norm(v, w, 1e-6)).max() < 1e-5
        assert torch.equal(out, out32)
        assert np.abs(nd.materialize("float32")[0].double().cpu().numpy() - plain.rms_norm(delta.sum(0), wd, 1e-5)).max() < 1e-5


@pytest.mark.parametrize("E,top,count,keep", [(12, 3, 4, 2), (8, 2, 2, 1), (6, 6, 1, 1), (9, 1, 3, 3), (256, 4, 128, 2)])
def test_experts_within_the_best_groups(E, top, count, keep):
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(E)
    for T in (1, 9, 70):
        h, router = rng.normal(size=(T, 40)), rng.normal(size=(E, 40))
        ids, weights, _ = plain.route(h, {"top": top, "groups": {"count": count, "keep": keep}}, router)
        x = torch.tensor(h, dtype=torch.float32, device="cuda")
        r = torch.tensor(router, dtype=torch.float32, device="cuda")
        got_ids, got_w, _ = ops.router_topk(x, r, None, top, False, "float32", groups=(count, keep))
        assert np.array_equal(got_ids.cpu().numpy(), ids)
        assert np.abs(got_w.double().cpu().numpy() - weights).max() < 1e-6
        routed = ops.route(x, r, None, top, False, 16, "float32", groups=(count, keep))
        assert np.array_equal(routed[0].cpu().numpy(), ids)


def test_delta_rule_kernels_with_a_state_carried_over(made):
    """The mixer's kernels against the plain function, the sequence cut in two runs so that the second starts from the
    first one's state and convolution inputs, and one more token through the decode step's single kernel; two sequences
    side by side in slots far apart."""
    from turboquant_cpp_amd.csrc import ops
    for case, layer in (("ragged", 1), ("ragged", 2), ("odd", 0)):
        _, cfg, w = made(case)
        m, p = cfg["layers"][layer]["mixer"], f"l{layer}.mix."
        H, G, D, V, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        ra, rg = w[p + "a1"].shape[0], w[p + "g1"].shape[0]
        dims = ops.DeltaDims(H, G, D, V, K, ra, rg)
        rng = np.random.default_rng(layer)
        lens, slots = (23, 1), (5, 2)
        hs = [rng.normal(size=(n + 10, cfg["width"])) for n in lens]
        want = [plain.channel_delta(h, m, w, p, 1e-5, return_state=True) for h in hs]
        dev = "cuda"
        f32 = lambda a: torch.tensor(np.ascontiguousarray(a), dtype=torch.float32, device=dev)
        state = torch.zeros((8, dims.state_floats + 3), dtype=torch.float32, device=dev)
        w_in = np.concatenate([w[p + n] for n in ("q", "k", "v", "b", "a1", "g1")])
        w_low = np.zeros((H * D + H * V, ra + rg))
        w_low[:H * D, :ra], w_low[H * D:, ra:] = w[p + "a2"], w[p + "g2"]
        conv = f32(np.concatenate([w[p + n] for n in ("q.conv", "k.conv", "v.conv")]))
        outs = [[], []]
        for run in range(3):
            parts = [h[:n] if run == 0 else h[n:n + 9] if run == 1 else h[n + 9:] for h, n in zip(hs, lens)]
            x = np.concatenate(parts)
            cu = np.cumsum([0] + [len(q) for q in parts])
            runs = {"cu_seqlens": torch.tensor(cu, dtype=torch.int32, device=dev),
                    "slots": torch.tensor(slots, dtype=torch.int32, device=dev), "decode": run == 2}
            slot_of_token = torch.tensor(np.repeat(slots, [len(q) for q in parts]), dtype=torch.int32, device=dev)
            proj = f32(x @ w_in.T)
            qn, kn, vc, beta, low = ops.delta_prep(proj, slot_of_token, state, conv, dims, "float32")
            if run == 2:
                assert ops.delta_decode_fits(dims)
                out = ops.delta_decode(qn, kn, vc, beta, low, f32(w_low), f32(w[p + "A_log"]), f32(w[p + "dt_bias"]),
                                       f32(w[p + "norm"]), 1e-5, proj, runs, state, dims, "float32")
            else:
                ag = f32(low.double().cpu().numpy() @ w_low.T)
                o = ops.delta_scan(qn, kn, vc, beta, ag, f32(w[p + "A_log"]), f32(w[p + "dt_bias"]), runs, state, dims, "float32")
                out = ops.delta_out(o, ag, f32(w[p + "norm"]), 1e-5, proj, runs, state, dims, "float32")
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


def test_a_conversation_with_state_and_chunks(made, tmp_path):
    """``Model.chat`` on a model with recurrent state and chunked groups: a turn that goes on runs only the new tokens; a
    history that parts from the cached tokens starts over (a state has no earlier value); a saved conversation (pages,
    rows of state, tokens) goes on in another model object with the same tokens."""
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
    assert info.returncode == 0 and "Felepel" in info.stdout and "max_positions" in info.stdout, info.stderr[-1000:]
    run = subprocess.run([quant, d, "-p", "5,17,3;8,1", "-n", "6", "-T", "0", "--rep-penalty", "1.0", "--dtype", "float32",
                          "--json", "-M"], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    with Model(d, dtype="float32", temperature=0.0, rep_penalty=1.0, max_tokens=6) as m:
        want = m.generate([[5, 17, 3], [8, 1]])
    got = [r["tokens"] for r in json.loads(run.stdout.strip().splitlines()[-1])]
    assert got == want
    c = subprocess.run([os.path.join(ROOT, "bin", "quant_c"), d, "-p", "5,17"], capture_output=True, text=True, timeout=300)
    assert c.returncode == 2 and "bin/quant runs this model" in c.stderr


def test_trace_runner_as_a_program(made, tmp_path):
    d, cfg, w = made("odd", seed=6)
    a, b = tokens(cfg, 90, 60), tokens(cfg, 41, 61)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:80], "want": [0, 41, 79]}, {"id": "b", "tokens": b[:40], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[80:81], "want": [0]}, {"id": "b", "tokens": b[40:], "want": [0]}], "end": ["b"]}]
    steps += [{"step": 2 + i, "entries": [{"id": "a", "tokens": [t], "want": [0] if i % 2 else []}], "end": ["a"] if i == 8 else []}
              for i, t in enumerate(a[81:])]
    out = tmp_path / "out"
    run = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "float32", "--out", str(out),
                          "--max-tokens", "256"], input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                         capture_output=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    wa, wb = plain.forward(cfg, w, a), plain.forward(cfg, w, b)
    V = cfg["vocab"]
    read = lambda i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V)
    check(read(0), wa[[0, 41, 79]], what="step 0")
    check(read(1), np.stack([wa[80], wb[40]]), what="step 1")
    for i in range(9):
        if i % 2:
            check(read(2 + i), wa[81 + i:82 + i], what=f"step {2 + i}")
        else:
            assert not (out / f"{2 + i}.f32").exists()
