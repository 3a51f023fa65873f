"""Megozen without a GPU: configuration, plan, frequency table, and the plain implementation's own properties."""
import copy
import math

import numpy as np
import pytest

import sprout_lm_amd as S
from sprout_lm_amd.config.base import ConfigError
from sprout_lm_amd.registry import build_model_plan
from tests import megozen_helpers as MH
from tests.plain import megozen_plain as M


@pytest.mark.parametrize("name", sorted(MH.CONFIGS))
def test_config_round_trip(name):
    cfg = S.config_from_dict(MH.CONFIGS[name])
    assert cfg.architecture == "Megozen"
    again = S.config_from_dict(cfg.to_dict())
    assert again == cfg
    assert cfg.to_dict() == S.config_from_dict(copy.deepcopy(cfg.to_dict())).to_dict()
    assert cfg.vocab_size == MH.CONFIGS[name]["vocab"] and cfg.hidden_size == MH.CONFIGS[name]["width"]


def test_config_refuses_what_it_cannot_be():
    def broken(edit):
        raw = copy.deepcopy(MH.GENERAL)
        edit(raw)
        with pytest.raises(ConfigError):
            S.config_from_dict(raw)
    broken(lambda r: r["layers"][0].update(type="convolution"))
    broken(lambda r: r["layers"][0]["mlp"]["router"].update(top=6))
    broken(lambda r: r["layers"][0]["mlp"].update(kind="dense"))
    broken(lambda r: r["layers"][0].update(weights_of=0))
    broken(lambda r: r["layers"][2].update(weights_of=7))
    broken(lambda r: (r["layers"][0].update(weights_of=2)))          # 0 -> 2 -> 0
    broken(lambda r: r["layers"][1]["mixer"].pop("kv_rank"))
    broken(lambda r: r["layers"][1]["mixer"]["rot"].update(dims=7))
    broken(lambda r: r["norm"].pop("eps"))
    broken(lambda r: r.pop("vocab"))
    broken(lambda r: r.update(layers=[]))


def test_plan_names_shapes_and_slots():
    cfg = S.config_from_dict(MH.VARIED)
    plan = build_model_plan(cfg)
    expected = plan.expected_tensors()
    assert tuple(expected["embed"].shape) == (300, 128) and tuple(expected["bigram"].shape) == (65, 128)
    assert tuple(expected["head"].shape) == (300, 128) and tuple(expected["final.norm"].shape) == (128,)
    assert tuple(expected["l0.mix.q"].shape) == (4 * 48, 128) and tuple(expected["l0.mix.dkv"].shape) == (64, 128)
    assert tuple(expected["l0.mix.uk"].shape) == (4 * 32, 48) and tuple(expected["l0.mix.uv"].shape) == (4 * 16, 48)
    assert tuple(expected["l0.mix.g"].shape) == (4, 128) and tuple(expected["l0.mix.o"].shape) == (128, 64)
    assert tuple(expected["l3.mix.uv"].shape) == (2 * 24, 32) and tuple(expected["l3.mix.dkv.norm"].shape) == (32,)
    assert tuple(expected["l3.mlp.e5.down"].shape) == (128, 40) and tuple(expected["l3.mlp.shared.up"].shape) == (72, 128)
    assert tuple(expected["l0.mlp.router.b"].shape) == (4,) and "l0.mlp.shared.gate" not in expected
    assert not any(n.startswith("l2.") for n in expected), "a layer that runs with another's tensors has none"
    assert not any(n.startswith("l1.mlp") or n.startswith("l1.norm2") for n in expected)
    # the run order: layers 1 and 2 are two calls of one layer, each with a cache slot of its own; the embedding's slot last
    assert [(c.layer, c.cache_slot) for c in plan.schedule] == [(0, 0), (1, 1), (1, 2), (2, 3)]
    assert plan.embedding_slot == 4
    parts = plan.instantiate()
    windows = [spec.window for spec in parts.cache_slot_specs[:4]]
    assert windows == [70, None, None, 33]
    assert [spec.head_dim for spec in parts.cache_slot_specs[:4]] == [64, 64, 64, 64]
    assert not parts.prefix_sharing       # the token before a step's first one is state of the request


def test_a_chain_of_shared_tensors_resolves_to_its_owner():
    cfg = S.config_from_dict(MH.MANY_HEADS)
    assert [cfg.source_of(i) for i in range(3)] == [0, 0, 0]
    plan = build_model_plan(cfg)
    assert len(plan.layers) == 1 and [(c.layer, c.cache_slot) for c in plan.schedule] == [(0, 0), (0, 1), (0, 2)]


@pytest.mark.parametrize("dims,base,scaling", [(8, 10000.0, (4.0, 64, 16.0, 2.0)), (16, 500.0, None),
                                               (32, 100000.0, (8.0, 32, 4.0, 0.5)), (64, 1e6, (40.0, 4096, 32.0, 1.0)),
                                               (2, 10.0, (1.5, 8, 2.0, 1.0))])
def test_frequency_table_of_the_rotary_part(dims, base, scaling):
    from sprout_lm_amd.parts.rotary import InterleavedRotary
    named = dict(zip(("factor", "original", "fast", "slow"), scaling)) if scaling else None
    part = InterleavedRotary(dims, base, named)
    want, magnitude = M.yarn_frequencies({"dims": dims, "base": base, "scaling": named})
    assert np.allclose(part.frequencies().numpy(), want, rtol=1e-14, atol=0)
    assert math.isclose(part.magnitude, magnitude, rel_tol=1e-15)
    if scaling is None:
        assert part.magnitude == 1.0 and np.allclose(want, base ** (-2.0 * np.arange(dims // 2) / dims))
    else:       # slow pairs are divided by the factor, fast pairs are left alone, nothing leaves that range
        plain = base ** (-2.0 * np.arange(dims // 2) / dims)
        assert np.all(want <= plain * (1 + 1e-12)) and np.all(want >= plain / scaling[0] * (1 - 1e-12))


# ------------------------------------------------------------------ the plain implementation's own properties
def test_plain_rotation_depends_on_the_distance_only():
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}}
    rng = np.random.default_rng(0)
    q, k = rng.normal(size=(1, 12)), rng.normal(size=(1, 12))
    def score(i, j):
        return float(M.rotate_interleaved(q, [i], rot)[0] @ M.rotate_interleaved(k, [j], rot)[0])
    assert math.isclose(score(40, 33), score(1007, 1000), rel_tol=1e-9)
    assert not math.isclose(score(40, 33), score(40, 31), rel_tol=1e-3)
    turned = M.rotate_interleaved(q, [5], rot)[0]
    assert np.array_equal(turned[8:], q[0, 8:])       # what lies behind rot.dims passes unchanged
    _, magnitude = M.yarn_frequencies(rot)
    assert math.isclose(np.hypot(turned[0], turned[1]), magnitude * np.hypot(q[0, 0], q[0, 1]), rel_tol=1e-12)


def test_plain_window_and_routing():
    seen = M.window_mask(6, 3)
    assert seen[5].tolist() == [False, False, False, True, True, True] and seen[1].tolist() == [True, True] + [False] * 4
    assert M.window_mask(4, None)[3].all()
    logits = np.asarray([[0.1, 2.0, 2.0, -1.0, 1.5]])
    chosen, weight = M.route(logits, 3)
    assert chosen.tolist() == [[1, 2, 4]]
    e = np.exp(np.asarray([2.0, 2.0, 1.5]) - 2.0)
    assert np.allclose(weight[0], e / e.sum())
    assert M.bigram_rows([4, 9, 9, 0], 7, 3, 5).tolist() == [7, (4 * 3 + 9 * 5) % 7, (9 * 3 + 9 * 5) % 7, (9 * 3) % 7]


def test_plain_forward_is_causal_and_forgets_beyond_its_windows():
    cfg = copy.deepcopy(MH.ONE_LAYER)
    weights = {n: a.astype(np.float64) for n, a in MH.random_weights(cfg, 3).items()}
    tokens = MH.random_tokens(cfg["vocab"], 60, 1)
    whole = M.forward(weights, cfg, tokens)
    assert np.allclose(whole[:40], M.forward(weights, cfg, tokens[:40]), atol=1e-6)
    other = list(tokens)
    other[10] = (other[10] + 1) % cfg["vocab"]
    changed = M.forward(weights, cfg, other)
    window = cfg["layers"][0]["mixer"]["mask"]["size"]
    # one layer: position i reads keys i - window + 1 .. i; token 10 also enters the pair row of position 11
    assert np.abs(changed[11 + window:] - whole[11 + window:]).max() < 1e-6
    assert np.abs(changed[10 + window - 1] - whole[10 + window - 1]).max() > 1e-4
