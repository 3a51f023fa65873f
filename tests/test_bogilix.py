"""Bogilix without a GPU: the configuration's round trips and refusals, the plan's tensors and cache slots, and
properties of the plain implementation itself."""
import copy

import numpy as np
import pytest

import sprout_lm_amd as S
from sprout_lm_amd.config.base import ConfigError
from sprout_lm_amd.registry import build_model_plan
from tests import bogilix_helpers as BH
from tests.plain import bogilix_plain as B


@pytest.mark.parametrize("name", sorted(BH.CONFIGS))
def test_configuration_round_trip(name):
    raw = BH.CONFIGS[name]
    cfg = S.config_from_dict(raw)
    assert cfg.architecture == "Bogilix" and cfg.to_dict() == raw
    assert S.config_from_dict(cfg.to_dict()) == cfg
    assert cfg.vocab_size == raw["vocab"] and cfg.hidden_size == raw["width"]


def broken(path, value, base="general"):
    raw = copy.deepcopy(BH.CONFIGS[base])
    at = raw
    for key in path[:-1]:
        at = at[key]
    if value is KeyError:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    return raw


@pytest.mark.parametrize("path,value", [
    (("vocab",), 0), (("width",), "wide"), (("norm",), None), (("layers",), []), (("layers", 0, "type"), "attention_3"),
    (("layers", 0, "mixer", "heads"), 3), (("layers", 0, "mixer", "rot"), KeyError), (("layers", 0, "mixer", "rot", "dims"), 7),
    (("layers", 0, "mixer", "rot", "dims"), 40), (("layers", 1, "mixer", "softcap"), KeyError), (("layers", 1, "mixer", "softcap"), -1.0),
    (("layers", 0, "mixer", "mask"), KeyError), (("layers", 0, "mixer", "scale"), 0), (("layers", 0, "mlp", "kind"), "sparse"),
    (("layers", 1, "mlp", "router", "groups", "count"), 3), (("layers", 1, "mlp", "router", "groups", "keep"), 5),
    (("layers", 1, "mlp", "router", "top"), 5), (("layers", 1, "mlp", "expert", "limit"), KeyError),
    (("layers", 2, "mixer", "vdim"), 48), (("layers", 1, "mixer", "v_mix"), "yes"),
])
def test_configuration_refusals(path, value):
    with pytest.raises(ConfigError):
        S.config_from_dict(broken(path, value))


def test_router_keys_that_may_be_left_out():
    raw = copy.deepcopy(BH.CONFIGS["general"])
    router = raw["layers"][1]["mlp"]["router"]
    del router["identity"], router["groups"]
    mlp = S.config_from_dict(raw).layers[1].mlp
    assert (mlp.identity, mlp.groups, mlp.keep) == (0, 1, 1)


def test_plan_names_every_tensor_and_cache_slot():
    from sprout_lm_amd.cache.spec import PagedKVSpec
    from sprout_lm_amd.parts.sink_attention import padded_width
    plan = build_model_plan(S.config_from_dict(BH.ODD))
    names = plan.expected_tensors()
    shapes = {n: tuple(s.shape) for n, s in names.items()}
    assert shapes["embed"] == (77, 100) and shapes["head"] == (77, 100) and shapes["final.norm.b"] == (100,)
    assert shapes["l0.mix.q"] == (60, 100) and shapes["l0.mix.v"] == (18, 100) and shapes["l0.mix.o"] == (100, 18)
    assert "l0.mix.q.b" not in names and "l0.mix.vmix" not in names and shapes["l0.mix.sink"] == (3,)
    assert shapes["l1.mix.q.b"] == (72,) and shapes["l1.mix.k.norm"] == (24,) and shapes["l1.mix.vmix"] == ()
    assert shapes["l0.mlp.router"] == (6, 100) and shapes["l0.mlp.correction"] == (6,) and "l0.mlp.e5.gate" not in names
    assert shapes["l0.mlp.e4.down"] == (100, 28) and shapes["l0.mlp.shared.sg"] == (1, 100) and shapes["l0.mlp.shared.up"] == (20, 100)
    assert shapes["l1.mlp.gate"] == (28, 100) and not any(n.startswith("l2.mlp") or n.startswith("l2.norm2") for n in names)
    assert "l3.mlp.shared.gate" not in names and shapes["l3.mlp.router"] == (9, 100)
    parts = plan.instantiate()
    specs = parts.cache_slot_specs
    assert len(specs) == 4 and all(isinstance(s, PagedKVSpec) for s in specs)
    # keys and values at one common width; what a block of the mask no longer reaches may be given back
    assert [(s.kv_heads, s.head_dim, s.window) for s in specs] == [(3, padded_width(20, 6), 1), (2, padded_width(12, 10), 5),
                                                                  (2, padded_width(6, 10), 37), (2, padded_width(16, 10), 37)]
    assert parts.prefix_sharing and parts.graph_safe and parts.graph_safe_portions
    mixers = [b.parts()["mixer"] for b in parts.blocks]
    assert [m.value_mix for m in mixers] == [None, "first", "blend", "blend"]
    assert padded_width(40, 64) == 64 and padded_width(20, 6) == 32 and padded_width(100, 7) == 128 and padded_width(130, 8) == 144


def test_plain_blocks_sinks_and_cap():
    """What the plain functions themselves promise: a query never sees a key of another block; a sink far above the
    scores empties the output and one far below is the plain softmax; the cap bounds every score; the rotation's scores
    depend on the distance alone, and only the first numbers of a head turn."""
    rng = np.random.default_rng(1)
    assert B.block_mask(7, 3).astype(int).tolist() == [[1, 0, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0, 0],
                                                       [0, 0, 0, 1, 0, 0, 0], [0, 0, 0, 1, 1, 0, 0], [0, 0, 0, 1, 1, 1, 0],
                                                       [0, 0, 0, 0, 0, 0, 1]]
    q, k, v = rng.normal(0, 1, (12, 2, 8)), rng.normal(0, 1, (12, 1, 8)), rng.normal(0, 1, (12, 1, 5))
    base = B.attend(q, k, v, 2, 1, 0.3, 4, [-60.0, -60.0], None, store=lambda a: a).reshape(12, 2, 5)
    moved = k.copy(); moved[3] += 5.0; v2 = v.copy(); v2[3] -= 9.0
    other = B.attend(q, moved, v2, 2, 1, 0.3, 4, [-60.0, -60.0], None, store=lambda a: a).reshape(12, 2, 5)
    assert np.abs(base[4:] - other[4:]).max() == 0 and np.abs(base[3] - other[3]).max() > 0.1
    np.testing.assert_allclose(base[0], np.broadcast_to(v[0], (2, 5)), atol=1e-12)      # the first token sees itself alone
    assert np.abs(B.attend(q, k, v, 2, 1, 0.3, 4, [80.0, 80.0], None, store=lambda a: a)).max() < 1e-20
    half = B.attend(q[:1], k[:1], v[:1], 2, 1, 0.3, 4, [float(0.3 * q[0, 0] @ k[0, 0]), -60.0], None, store=lambda a: a).reshape(2, 5)
    np.testing.assert_allclose(half[0], 0.5 * v[0, 0], atol=1e-12)                       # a sink equal to the one score: a half
    capped = B.attend(100 * q, k, v, 2, 1, 0.3, 12, [0.0, 0.0], 2.0, store=lambda a: a).reshape(12, 2, 5)
    assert np.isfinite(capped).all() and np.abs(capped - B.attend(100 * q, k, v, 2, 1, 0.3, 12, [0.0, 0.0], None, store=lambda a: a).reshape(12, 2, 5)).max() > 1e-3
    x = rng.normal(0, 1, (1, 1, 10))
    a, b = B.turn_halves(np.repeat(x, 2, 0), [3, 103], 6, 50.0), B.turn_halves(np.repeat(rng.normal(0, 1, (1, 1, 10)), 2, 0), [10, 110], 6, 50.0)
    assert abs(float(a[0, 0, :6] @ b[0, 0, :6]) - float(a[1, 0, :6] @ b[1, 0, :6])) < 1e-12
    assert (a[:, 0, 6:] == x[0, 0, 6:]).all()
    turned = B.turn_halves(np.asarray([[[1.0, 0, 0, 0, 7.0]]]), [1], 4, 100.0)[0, 0]
    np.testing.assert_allclose(turned, [np.cos(1.0), 0.0, np.sin(1.0), 0.0, 7.0], atol=1e-12)   # number 0 turns with number 2


def test_plain_routing_rule():
    """The correction moves the choice and not the weights; only the best groups are open, also where every sum is
    negative; the lower index wins a tie; the weights are not renormalised."""
    z = np.log(np.asarray([[0.1, 0.2, 0.3, 0.25, 0.1, 0.05]]))
    ids, w = B.route(z, np.zeros(6), 2, 1, 1, 2.0)
    assert ids.tolist() == [[2, 3]] and np.allclose(w, [[0.6, 0.5]])
    ids, w = B.route(z, np.asarray([0.5, 0, 0, 0, 0, 0]), 2, 1, 1, 1.0)
    assert ids.tolist() == [[0, 2]] and np.allclose(w, [[0.1, 0.3]])
    ids, _ = B.route(z, np.zeros(6), 2, 3, 1, 1.0)          # groups (0,1) (2,3) (4,5): the best is (2,3)
    assert ids.tolist() == [[2, 3]]
    ids, _ = B.route(z, np.asarray([0.0, 0.0, -1.0, 0.0, 0.0, 0.0]) - 5.0, 2, 3, 1, 1.0)   # all negative: group (2,3) still wins by 0.25
    assert ids.tolist() == [[3, 2]]
    ids, _ = B.route(z, np.asarray([0.0, 0.05, -0.2, -0.2, 0.0, 0.0]), 3, 3, 2, 1.0)
    assert sorted(ids[0].tolist()) == [0, 1, 4]             # groups (0,1) and (4,5) stay; their three best
    ids, _ = B.route(np.zeros((1, 6)), np.zeros(6), 3, 3, 2, 1.0)
    assert ids.tolist() == [[0, 1, 2]]


def test_plain_identity_experts_and_shared_gate():
    rng = np.random.default_rng(2)
    f = BH.moe(2, 2, 4, 1, 1, 1.5, 6, 0.7, shared=(5, 0.9))
    w = {"router": rng.normal(0, 1, (4, 8)), "correction": np.zeros(4)}
    for e in range(2):
        w.update({f"e{e}.gate": rng.normal(0, 1, (6, 8)), f"e{e}.up": rng.normal(0, 1, (6, 8)), f"e{e}.down": rng.normal(0, 1, (8, 6))})
    w.update({"shared.gate": rng.normal(0, 1, (5, 8)), "shared.up": rng.normal(0, 1, (5, 8)), "shared.down": rng.normal(0, 1, (8, 5)),
              "shared.sg": rng.normal(0, 1, (1, 8))})
    h = rng.normal(0, 1, (3, 8))
    out = B.routed_ff(w, "", f, h, store=lambda a: a)
    z = h @ w["router"].T
    s = np.exp(z) / np.exp(z).sum(-1, keepdims=True)
    want = np.zeros_like(out)
    for t in range(3):
        for e in range(2):
            want[t] += 1.5 * s[t, e] * B.expert(w, f"e{e}.", h[t:t + 1], 0.7, store=lambda a: a)[0]
        want[t] += 1.5 * (s[t, 2] + s[t, 3]) * h[t]
        want[t] += B.sigmoid(h[t] @ w["shared.sg"][0]) * B.expert(w, "shared.", h[t:t + 1], 0.9, store=lambda a: a)[0]
    np.testing.assert_allclose(out, want, atol=1e-12)
    g = np.asarray([[-3.0, 0.2, 5.0]])
    y = B.expert({"gate": np.eye(3), "up": -2 * np.eye(3), "down": np.eye(3)}, "", g, 1.0, store=lambda a: a)[0]
    gc, uc = np.minimum(g[0], 1.0), np.clip(-2 * g[0], -1.0, 1.0)
    np.testing.assert_allclose(y, gc / (1 + np.exp(-1.702 * gc)) * (uc + 1), atol=1e-12)


def test_plain_causality_and_blend():
    """A later token never changes an earlier logit; a token of another block changes a later logit only through the
    blended values and feed-forwards of its own position, that is: not at all."""
    import tempfile
    with tempfile.TemporaryDirectory() as root:
        folder = BH.make_folder(root, "odd")
        tokens = BH.random_tokens(77, 40, 3)
        full = BH.plain_logits(folder, "float32", tokens)
        short = BH.plain_logits(folder, "float32", tokens[:25])
        assert np.abs(full[:25] - short).max() < 1e-5
        changed = list(tokens); changed[2] = (changed[2] + 1) % 77
        # the longest block of this model has 37 positions: position 2 lies in block 0, position 39 in block 1 of every layer
        other = BH.plain_logits(folder, "float32", changed)
        assert np.abs(other[39] - full[39]).max() < 1e-5 and np.abs(other[5] - full[5]).max() > 1e-4
