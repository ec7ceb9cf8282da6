"""What of the Taminex design can be checked without a GPU: its config.json, its plan and tensor table, which schedule
entry reads whose latents, and the plain implementation's mechanisms against small cases worked out by hand."""
import copy

import numpy as np
import pytest

import plain_taminex as plain
from taminex_cases import CASES, attention, config, delta, dense, latent, random_case, tensors
from turboquant_cpp_amd.config import ConfigError, config_from_dict
from turboquant_cpp_amd.engine.model import CausalLM


@pytest.mark.parametrize("case", sorted(CASES))
def test_the_plan_reads_exactly_the_folder_s_tensors(case):
    cfg_json = CASES[case]
    w = tensors(cfg_json, 0)
    arch, cfg = config_from_dict(cfg_json)
    model = CausalLM(arch.plan(cfg), "float32", config=cfg)
    table = model.tensor_table()
    assert set(table) == set(w)
    for name, (shape, _role) in table.items():
        assert tuple(shape) == w[name].shape, name
    # a layer on another's latents is a schedule entry that reads the other entry's cache; every other entry has its own
    assert len(model.schedule) == len(cfg_json["layers"])
    for entry, layer in zip(model.schedule, cfg_json["layers"]):
        assert entry.cache_of == layer["mixer"].get("kv_from")
    assert arch.config_from_json(arch.config_to_json(cfg)) == cfg


@pytest.mark.parametrize("seed", range(12))
def test_plans_of_sizes_of_many_kinds(seed):
    cfg_json = random_case(seed)
    arch, cfg = config_from_dict(cfg_json)
    model = CausalLM(arch.plan(cfg), "bfloat16", config=cfg)
    assert set(model.tensor_table()) == set(tensors(cfg_json, seed))


def test_what_config_json_may_leave_out_and_may_not():
    base = config(32, 40, [(attention(2, 1, 16, 16, rot=8), dense(24)), (delta(2, 2, 8, 8), None),
                           (latent(2, 8, 8, 12), None), (latent(1, 4, 4, 12, kv_from=2), dense(8))],
                  logit_scale=2.0, logit_softcap=9.0)
    _, cfg = config_from_dict(base)
    assert cfg.logit_scale == 2.0 and cfg.logit_softcap == 9.0 and cfg.layers[1].mlp is None
    assert cfg.layers[0].mixer.rot_dims == 8 and cfg.layers[3].mixer.kv_from == 2 and cfg.layers[2].mixer.kv_from is None
    free = copy.deepcopy(base)
    del free["logit_scale"], free["logit_softcap"], free["layers"][0]["mixer"]["rot"]
    _, c2 = config_from_dict(free)
    assert c2.logit_scale == 1.0 and c2.logit_softcap is None and c2.layers[0].mixer.rot_dims == 0
    for path, value, message in [(("width",), None, "width"), (("vocab",), None, "vocab"), (("norm",), None, "norm"),
                                 (("layers", 0, "mixer", "scale"), None, "scale"),
                                 (("layers", 0, "type"), "conv", "not implemented"),
                                 (("layers", 0, "mixer", "kv_heads"), 3, "multiple"),
                                 (("layers", 0, "mixer", "rot", "dims"), 7, "even"),
                                 (("layers", 0, "mixer", "rot", "dims"), 18, "at most"),
                                 (("layers", 0, "mlp", "kind"), "moe", "not implemented"),
                                 (("layers", 1, "mixer", "conv"), None, "conv"),
                                 (("layers", 2, "mixer", "kv_rank"), None, "kv_rank"),
                                 (("layers", 3, "mixer", "kv_rank"), 16, "kv_rank"),
                                 (("layers", 3, "mixer", "kv_from"), 1, "keeps no latents"),
                                 (("layers", 3, "mixer", "kv_from"), 3, "another layer"),
                                 (("layers", 2, "mixer", "kv_from"), 3, "keeps no latents")]:
        bad = copy.deepcopy(base)
        at = bad
        for k in path[:-1]:
            at = at[k]
        if value is None:
            del at[path[-1]]
        else:
            at[path[-1]] = value
        with pytest.raises(ConfigError, match=message):
            config_from_dict(bad)


def test_plain_norm_has_eps_inside_the_root():
    y = np.array([[3.0, 4.0]])
    assert np.allclose(plain.rms_norm(y, np.array([2.0, 0.5]), 0.5), y / np.sqrt(12.5 + 0.5) * [2.0, 0.5])


def test_plain_sink_counts_once_and_has_no_value():
    scores = np.array([[1.0, 9.0], [2.0, 0.5]])
    p = plain.causal_softmax(scores, 0, sink=0.25)
    assert np.allclose(p[0], [np.exp(1.0) / (np.exp(1.0) + np.exp(0.25)), 0.0])
    z = np.exp(2.0) + np.exp(0.5) + np.exp(0.25)
    assert np.allclose(p[1], [np.exp(2.0) / z, np.exp(0.5) / z])
    assert np.allclose(plain.causal_softmax(scores, 0, sink=-1e9), plain.causal_softmax(scores, 0))
    assert np.allclose(plain.causal_softmax(scores, 0).sum(1), 1.0)
    # a large sink takes nearly all of the weight: the row's output shrinks towards nothing
    assert plain.causal_softmax(scores, 0, sink=30.0).sum(1).max() < 1e-8


def test_plain_rotation_turns_neighbouring_pairs_of_the_first_dimensions():
    x = np.arange(1.0, 9.0).reshape(1, 1, 8)
    out = plain.rotate_pairs(np.repeat(x, 3, axis=0), np.array([0.0, 1.0, 5.0]), 4, 100.0)
    assert np.allclose(out[0], x[0]) and np.allclose(out[:, :, 4:], x[:, :, 4:])
    for row, p in ((1, 1.0), (2, 5.0)):
        for i, f in enumerate((1.0, 100.0 ** -0.5)):
            u, v, a = x[0, 0, 2 * i], x[0, 0, 2 * i + 1], p * f
            assert np.allclose(out[row, 0, 2 * i:2 * i + 2], [u * np.cos(a) - v * np.sin(a), v * np.cos(a) + u * np.sin(a)])
    # a score depends on the distance of the two positions only
    rng = np.random.default_rng(0)
    q, k = rng.normal(size=(1, 1, 8)), rng.normal(size=(1, 1, 8))
    at = lambda pq, pk: float(np.sum(plain.rotate_pairs(q, np.array([pq]), 6, 50.0) * plain.rotate_pairs(k, np.array([pk]), 6, 50.0)))
    assert abs(at(9.0, 2.0) - at(307.0, 300.0)) < 1e-9 and abs(at(9.0, 2.0) - at(9.0, 3.0)) > 1e-3


def test_plain_convolution_s_last_column_is_the_present_token():
    x = np.array([[1.0], [10.0], [100.0], [1000.0]])
    taps = np.array([[3.0, 2.0, 1.0]])
    assert plain.short_convolution(x, taps)[:, 0].tolist() == [1.0, 12.0, 123.0, 1230.0]


def test_plain_delta_rule_by_hand_and_carried_over():
    cfg = CASES["delta_only"]
    w = tensors(cfg, 1)
    m = dict(cfg["layers"][0]["mixer"], conv=1)
    for n in ("q", "k", "v"):
        w[f"l0.mix.{n}.conv"] = w[f"l0.mix.{n}.conv"][:, -1:]
    h = np.random.default_rng(0).normal(size=(30, cfg["width"]))
    whole = plain.head_delta(h, m, w, "l0.mix.", 1e-5)
    first, S = plain.head_delta(h[:17], m, w, "l0.mix.", 1e-5, return_state=True)
    second = plain.head_delta(h[17:], m, w, "l0.mix.", 1e-5, state=S)
    assert np.abs(np.concatenate([first, second]) - whole).max() < 1e-12
    # one token from an empty state: S = beta k v^T whatever the decay, read out with q
    one, S1 = plain.head_delta(h[:1], m, w, "l0.mix.", 1e-5, return_state=True)
    p, D = "l0.mix.", m["dim"]
    k = plain.silu(h[:1] @ w[p + "k"].T * w[p + "k.conv"][:, 0]).reshape(m["kv_heads"], D)
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    v = plain.silu(h[:1] @ w[p + "v"].T * w[p + "v.conv"][:, 0]).reshape(m["heads"], m["vdim"])
    beta = plain.sigmoid(h[:1] @ w[p + "b"].T)[0]
    for head in range(m["heads"]):
        assert np.allclose(S1[head], beta[head] * np.outer(k[head // (m["heads"] // m["kv_heads"])], v[head]))


def test_plain_latents_may_stay_compressed():
    """q . (W_uk c) = (W_uk^T q) . c and sum_j p_j W_uv c_j = W_uv sum_j p_j c_j: attention over the latents themselves,
    with each head's key matrix taken into its query and its value matrix applied afterwards, is the same function."""
    cfg = CASES["latent_only"]
    w = tensors(cfg, 2)
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    H, D, V, R = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
    h = np.random.default_rng(1).normal(size=(11, cfg["width"]))
    c = plain.latent_of(h, w, p, 1e-5)
    want = plain.latent_attention(h, c, m, w, p)
    q = (h @ w[p + "q"].T).reshape(-1, H, D)
    heads = np.zeros((len(h), H, V))
    for head in range(H):
        folded = q[:, head] @ w[p + "uk"].reshape(H, D, R)[head]
        probs = plain.causal_softmax(folded @ c.T * m["scale"], 0)
        heads[:, head] = (probs @ c) @ w[p + "uv"].reshape(H, V, R)[head].T
    got = (heads.reshape(len(h), H * V) * plain.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T
    assert np.abs(got - want).max() < 1e-12


def test_plain_shared_latents_are_the_other_layer_s():
    cfg = CASES["shared_latent"]
    w = tensors(cfg, 3)
    toks = [5, 9, 2, 77, 31, 8]
    base = plain.forward(cfg, w, toks)
    changed = dict(w)
    changed["l0.mix.dkv.norm"] = w["l0.mix.dkv.norm"] * 1.5        # layer 0's latents, which layer 1 reads
    other = plain.forward(cfg, changed, toks)
    # layer 0's own softmax and values change with it, so take layer 0 out of the stream: its norm's weight to zero
    for ww in (w, changed):
        ww["l0.norm1"] = np.zeros_like(w["l0.norm1"])
    a, b = plain.forward(cfg, w, toks), plain.forward(cfg, changed, toks)
    assert np.abs(a - b).max() > 1e-3 and np.abs(base - other).max() > 1e-3


def test_plain_logits_are_scaled_and_then_capped():
    cfg = CASES["ff_only_behind_attention"]
    w = tensors(cfg, 4)
    toks = [3, 1, 4, 1, 5]
    free = dict(cfg, logit_scale=1.0)
    del free["logit_softcap"]
    raw = plain.forward(free, w, toks)
    assert np.allclose(plain.forward(cfg, w, toks), 8.0 * np.tanh(raw * 3.0 / 8.0))
