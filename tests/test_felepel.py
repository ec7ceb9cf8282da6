"""What of the Felepel design can be checked without a GPU: its config.json, its plan and tensor table, the cache's
books for chunks of positions, and the plain implementation against itself."""
import copy

import numpy as np
import pytest

import plain_felepel as plain
from felepel_cases import CASES, attention, config, delta, moe, tensors, tokens
from turboquant_cpp_amd.cache.paged import PagedCache
from turboquant_cpp_amd.config import ConfigError, config_from_dict
from turboquant_cpp_amd.engine.model import CausalLM
from turboquant_cpp_amd.parts.base import CacheNeed


def completed(cfg_json, w):
    arch, cfg = config_from_dict(cfg_json)
    return arch, arch.complete(cfg, {n: v.shape for n, v in w.items()})


@pytest.mark.parametrize("case", sorted(CASES))
def test_the_plan_reads_exactly_the_folder_s_tensors(case):
    w = tensors(CASES[case], 0)
    arch, cfg = completed(CASES[case], w)
    model = CausalLM(arch.plan(cfg), "float32", config=cfg)
    table = model.tensor_table()
    assert set(table) == set(w)
    for name, (shape, _role) in table.items():
        assert tuple(shape) == w[name].shape, name
    # a layer that names another's weights is another run of that layer, with a cache or state of its own
    assert len(model.schedule) == len(CASES[case]["layers"])
    assert all(e.cache_of is None for e in model.schedule)
    assert len(model.blocks) == sum(1 for l in CASES[case]["layers"] if l.get("weights_of") is None)
    assert arch.config_from_json(arch.config_to_json(cfg)) == cfg


def test_what_config_json_may_leave_out_and_may_not():
    base = config(32, 40, [(attention(2, 1, 16, 16), moe(4, 2, 8, 2, 1)), (delta(2, 2, 8, 8), None)])
    arch, cfg = config_from_dict(base)
    assert cfg.layers[0].mixer.chunk == 40 and cfg.layers[0].mixer.softcap == 30.0 and cfg.layers[1].mlp is None
    free = copy.deepcopy(base)
    del free["layers"][0]["mixer"]["softcap"], free["layers"][0]["mixer"]["mask"], free["layers"][0]["mlp"]["router"]["groups"]
    _, c2 = config_from_dict(free)
    assert c2.layers[0].mixer.chunk is None and c2.layers[0].mixer.softcap is None and c2.layers[0].mlp.groups == 1
    with pytest.raises(ConfigError, match="ranks"):        # the delta rule's ranks come from the tensors
        arch.plan(cfg)
    for path, value, message in [(("width",), None, "width"), (("layers", 0, "mixer", "scale"), None, "scale"),
                                 (("layers", 0, "type"), "conv", "not implemented"),
                                 (("layers", 0, "mixer", "kv_heads"), 3, "multiple"),
                                 (("layers", 0, "mlp", "router", "groups", "count"), 3, "groups"),
                                 (("layers", 0, "mlp", "kind"), "dense", "not implemented"),
                                 (("layers", 1, "mixer", "conv"), None, "conv")]:
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
    ahead = copy.deepcopy(base)
    ahead["layers"].insert(0, {**ahead["layers"][1], "weights_of": 2})      # a layer may run the tensors of a later one
    _, c3 = config_from_dict(ahead)
    assert c3.layers[0].weights_of == 2 and c3.layers[0].type == "channel_delta"
    bad = copy.deepcopy(base)
    bad["layers"].append({**bad["layers"][0], "weights_of": 1})       # an attention layer with a delta layer's weights
    with pytest.raises(ConfigError, match="weights of layer 1"):
        config_from_dict(bad)


def test_a_chunked_group_gives_back_what_lies_before_the_next_token_s_chunk():
    need = CacheNeed(1, 16, chunk=100)
    cache = PagedCache([(need, None, None), (CacheNeed(1, 16), None, None)], max_tokens=1024, dtype=None, device=None)
    chunked = next(g for g in cache.groups if g.key.chunk == 100)
    plain_group = next(g for g in cache.groups if g.key.chunk is None)
    slot = cache.open()
    held = lambda g: [int(p) for p in np.nonzero(g.host_table[slot] >= 0)[0]]
    for n, want in ((150, [1, 2]), (49, [1, 2, 3]), (1, [3]), (100, [4]), (1, [4])):
        cache.reserve(slot, n)
        cache.commit(slot)      # lengths 150, 199, 200, 300, 301: the next token's chunk starts at 100, 100, 200, 300, 300
        assert held(chunked) == want, (cache.length(slot), held(chunked))
    assert held(plain_group) == [0, 1, 2, 3, 4]
    with pytest.raises(Exception):
        cache.truncate(slot, 250)       # position 250 would look at 200.., which is given back
    cache.close(slot)
    assert cache.pages_held() == {0: 0, 1: 0}


def test_plain_delta_rule_carries_its_state():
    """The plain recurrence run in one piece equals itself run from a state that it returned (the convolution's
    inputs aside, which this cut keeps by starting the second piece where the filter has no earlier input left)."""
    cfg = CASES["delta_only"]
    w = tensors(cfg, 1)
    m = dict(cfg["layers"][0]["mixer"], conv=1)
    for n in ("q", "k", "v"):
        w[f"l0.mix.{n}.conv"] = w[f"l0.mix.{n}.conv"][:, -1:]
    h = np.random.default_rng(0).normal(size=(30, cfg["width"]))
    whole = plain.channel_delta(h, m, w, "l0.mix.", 1e-5)
    first, S = plain.channel_delta(h[:17], m, w, "l0.mix.", 1e-5, return_state=True)
    second = plain.channel_delta(h[17:], m, w, "l0.mix.", 1e-5, state=S)
    assert np.abs(np.concatenate([first, second]) - whole).max() < 1e-12


def test_plain_choice_of_experts_within_groups():
    x = np.array([[1.0, 0.0]])
    router = np.array([[3.0, 0.0], [2.9, 0.0], [0.0, 0.0], [3.5, 0.0]])        # the logits of experts 0..3: 3, 2.9, 0, 3.5
    ids, weights, _ = plain.route(x, {"top": 2, "groups": {"count": 2, "keep": 1}}, router)
    assert ids[0].tolist() == [3, 2]        # the best expert's group wins, and its other member comes with it
    s = np.exp(router[:, 0])
    assert np.allclose(weights[0], s[[3, 2]] / s.sum())       # scores of the softmax over all, as they are
    ids, _, _ = plain.route(x, {"top": 2, "groups": {"count": 1, "keep": 1}}, router)
    assert ids[0].tolist() == [3, 0]
    ids, _, _ = plain.route(x, {"top": 2}, router)
    assert ids[0].tolist() == [3, 0]


def test_plain_chunks_count_from_position_zero():
    ok = plain.attention_scores_mask(7, 3)
    assert ok[2].tolist() == [True, True, True, False, False, False, False]
    assert ok[3].tolist() == [False, False, False, True, False, False, False]
    assert ok[6].tolist() == [False] * 6 + [True]
