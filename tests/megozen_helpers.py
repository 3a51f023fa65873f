"""Tiny Megozen configurations, model folders with weights of the tests' own making, and the plain side's logits."""
from __future__ import annotations

import copy
import json
import os

import numpy as np
import torch

from tests.plain import megozen_plain as M


def mixer(heads, dim, rot_dim, vdim, kv_rank, scale, window=None, base=10000.0, scaling=None):
    out = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
           "rot": {"base": base, "dims": rot_dim}}
    if window is not None:
        out["mask"] = {"size": window}
    if scaling is not None:
        out["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return out


def experts(n, top, ff, shared=None):
    out = {"kind": "moe", "router": {"experts": n, "top": top}, "expert": {"ff": ff}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def layer(mix, mlp=None, weights_of=None):
    out = {"type": "latent_attention", "mixer": copy.deepcopy(mix), "mlp": copy.deepcopy(mlp)}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def model(width, vocab, layers, bigram=(97, 31, 5), eps=1e-5):
    return {"architecture": "Megozen", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))}, "layers": layers}


# general: a key width (kv_rank + rot_dim = 28) that only the general attention kernels take; every size differs from
# every other; a window that is no multiple of a page; the third layer runs with the first one's tensors
_G = mixer(3, 24, 8, 40, 20, 0.4, window=37, scaling=(4.0, 64, 16.0, 2.0))
_GF = experts(5, 2, 48, shared=24)
GENERAL = model(96, 211, [layer(_G, _GF), layer(_G, _GF), layer(_G, _GF, weights_of=0)])
# matrix-core sizes (key width 64); windows 70, none and 33 in one model (three page pools); a layer without a
# feed-forward, run twice; as many experts as are chosen; one chosen expert; no frequency scaling in one layer
_A = mixer(4, 32, 16, 16, 48, 0.3, window=70, scaling=(2.5, 128, 8.0, 1.0))
_B = mixer(4, 32, 16, 16, 48, 0.3, window=None, base=500.0)
_C = mixer(2, 16, 32, 24, 32, 0.5, window=33, base=100000.0, scaling=(8.0, 32, 4.0, 0.5))
VARIED = model(128, 300, [layer(_A, experts(4, 4, 24)), layer(_B), layer(_B, weights_of=1),
                          layer(_C, experts(6, 1, 40, shared=72))], bigram=(64, 3, 1), eps=1e-6)
# more query heads than any group of the attention kernels holds; a window of exactly one page; a chain of shared tensors
_H = mixer(20, 8, 4, 12, 12, 0.6, window=16)
MANY_HEADS = model(80, 128, [layer(_H, experts(3, 2, 16, shared=16)), layer(_H, experts(3, 2, 16, shared=16), weights_of=0),
                             layer(_H, experts(3, 2, 16, shared=16), weights_of=1)], bigram=(1, 0, 0))
# one layer, routed experts: what the bfloat16 comparisons of routing use (no rounding of earlier layers before the router)
ONE_LAYER = model(64, 150, [layer(mixer(2, 16, 8, 16, 24, 0.5, window=29), experts(7, 3, 32, shared=20))], bigram=(50, 7, 11))
# as many experts as are chosen in every layer: nothing discrete for bfloat16 rounding to flip
ALL_CHOSEN = model(96, 211, [layer(_G, experts(3, 3, 32, shared=24)), layer(_G, experts(3, 3, 32, shared=24)),
                             layer(_G, experts(3, 3, 32, shared=24), weights_of=0)])

# sizes in no whole eights or sixteens anywhere (width 100, key width 22, head sizes 12 + 6, values of 10, experts of 28
# and 36); a window of one key, a window of five inside a page, and a layer that sees everything; a router without a
# shared expert beside one with; large multipliers in the pair table
_O1 = mixer(5, 12, 6, 10, 16, 0.7, window=1, base=300.0)
_O5 = mixer(5, 12, 6, 10, 16, 0.7, window=5, scaling=(3.0, 16, 4.0, 1.0))
_OA = mixer(3, 20, 2, 6, 30, 0.2, window=None, base=20.0, scaling=(1.5, 8, 2.0, 1.0))
ODD = model(100, 77, [layer(_O1, experts(3, 2, 28)), layer(_O5, experts(9, 4, 36, shared=28)), layer(_OA),
                      layer(_O5, experts(9, 4, 36, shared=28), weights_of=1)], bigram=(13, 2 ** 31 + 11, 2 ** 20 + 3), eps=1e-3)

CONFIGS = {"odd": ODD, "general": GENERAL, "varied": VARIED, "many_heads": MANY_HEADS, "one_layer": ONE_LAYER, "all_chosen": ALL_CHOSEN}
PAGE = {"odd": 16, "general": 16, "varied": 16, "many_heads": 8, "one_layer": 4, "all_chosen": 16}
SEED = {"odd": 4, "general": 5, "varied": 6, "many_heads": 7, "one_layer": 8, "all_chosen": 9}


def random_weights(cfg: dict, seed: int) -> dict:
    """name -> float32 array for every tensor the configuration needs (shapes asked from the engine's plan, values
    the tests' own): tables N(0, 1), matrices N(0, 0.08), norm weights 1 + N(0, 0.1), router biases N(0, 0.3)."""
    import sprout_lm_amd as S
    from sprout_lm_amd.registry import build_model_plan
    expected = build_model_plan(S.config_from_dict(cfg)).expected_tensors()
    rng = np.random.default_rng(seed)
    out = {}
    for name in sorted(expected):
        shape = tuple(expected[name].shape)
        last = name.split(".")[-1]
        if name in ("embed", "bigram"):
            a = rng.normal(0.0, 1.0, shape)
        elif last in ("norm", "norm1", "norm2"):
            a = 1.0 + rng.normal(0.0, 0.1, shape)
        elif name.endswith("router.b"):
            a = rng.normal(0.0, 0.3, shape)
        elif name.endswith(".router"):
            a = rng.normal(0.0, 0.4, shape)
        else:
            a = rng.normal(0.0, 0.08, shape)
        out[name] = M.bf16_round(a.astype(np.float32))
    return out


def write_folder(folder: str, cfg: dict, weights: dict) -> str:
    from sprout_lm_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      {n: torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16) for n, a in weights.items()})
    return folder


def make_folder(root: str, name: str) -> str:
    folder = os.path.join(root, "megozen_" + name)
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        write_folder(folder, CONFIGS[name], random_weights(CONFIGS[name], SEED[name]))
    return folder


_MODELS: dict = {}
_LOGITS: dict = {}


def plain_logits(folder: str, dtype: str, tokens) -> np.ndarray:
    """The plain implementation's logits at every position of `tokens`."""
    key = (folder, dtype, tuple(tokens))
    if key not in _LOGITS:
        if folder not in _MODELS:
            _MODELS[folder] = M.load_folder(folder)
        cfg, w = _MODELS[folder]
        _LOGITS[key] = M.forward(w, cfg, list(tokens), store=M.bf16_round if dtype == "bfloat16" else M.f32)
    return _LOGITS[key]


def tolerance(dtype: str, ref: np.ndarray) -> float:
    """Bound of |engine - plain| on a row of logits: float32 sums against float64 sums, or one-unit flips of the
    bfloat16 roundings that both sides make at the same places."""
    return (2e-5 if dtype == "float32" else 3e-2) * max(1.0, float(np.abs(ref).max()))


def random_tokens(vocab: int, n: int, seed: int, avoid=()) -> list[int]:
    allowed = np.asarray([t for t in range(vocab) if t not in set(avoid)])
    return [int(t) for t in allowed[np.random.default_rng(seed).integers(0, len(allowed), n)]]
