"""Tiny Bogilix configurations, model folders with weights of the tests' own making, and the plain side's logits."""
from __future__ import annotations

import copy
import json
import os

import numpy as np
import torch

from tests.plain import bogilix_plain as B


def rotary(heads, kv_heads, dim, vdim, scale, chunk, dims, base=10000.0, v_mix=False):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                                           "mask": {"size": chunk}, "rot": {"dims": dims, "base": base}, "v_mix": v_mix}}


def normed(heads, kv_heads, dim, vdim, scale, chunk, softcap, v_mix=False):
    return {"type": "attention_2", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                                             "mask": {"size": chunk}, "softcap": softcap, "v_mix": v_mix}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, groups, keep, scale, ff, limit, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
           "router": {"experts": experts, "identity": identity, "top": top, "scale": scale, "groups": {"count": groups, "keep": keep}}}
    if shared is not None:
        out["shared"] = {"ff": shared[0], "limit": shared[1]}
    return out


def layer(mix, mlp=None):
    out = copy.deepcopy(mix)
    out["mlp"] = copy.deepcopy(mlp)
    return out


def model(width, vocab, layers, eps=1e-5):
    return {"architecture": "Bogilix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


# no size in whole eights or sixteens; blocks of one position and of five; a layer without a feed-forward; the first
# blending layer is not the first layer; groups of which some stay shut, an identity expert, experts without a shared one
ODD = model(100, 77, [
    layer(rotary(3, 3, 20, 6, 0.4, 1, 8, base=300.0), moe(5, 1, 3, 3, 2, 1.5, 28, 0.8, shared=(20, 1.2))),
    layer(normed(6, 2, 12, 10, 0.3, 5, 7.0, v_mix=True), dense(28)),
    layer(normed(4, 2, 6, 10, 0.9, 37, 2.5, v_mix=True)),
    layer(rotary(2, 2, 16, 10, 0.25, 37, 16, base=50.0, v_mix=True), moe(9, 0, 4, 1, 1, 0.7, 36, 2.0)),
], eps=1e-3)
# sizes the matrix-core kernels take: keys narrower than values and wider, part of a head turning, 32 query heads over
# one key/value head (more than a block of the one-query kernel holds), blocks of 16 to 70 positions
GENERAL = model(128, 300, [
    layer(rotary(4, 2, 32, 64, 0.2, 48, 16), dense(96)),
    layer(normed(8, 1, 64, 32, 0.15, 70, 30.0, v_mix=True), moe(6, 2, 2, 4, 2, 2.5, 64, 1.0, shared=(64, 2.0))),
    layer(rotary(4, 1, 64, 32, 0.125, 33, 64, base=250.0, v_mix=True), moe(6, 2, 2, 4, 2, 2.5, 64, 1.0, shared=(64, 2.0))),
    layer(normed(32, 1, 16, 32, 0.3, 16, 4.0, v_mix=True), dense(96)),
])
# every router output chosen in every layer: nothing discrete for bfloat16 rounding to flip
ALL_CHOSEN = model(96, 211, [
    layer(normed(6, 2, 16, 32, 0.3, 40, 20.0, v_mix=True), moe(3, 1, 4, 2, 2, 1.2, 32, 1.5, shared=(24, 1.0))),
    layer(rotary(6, 2, 32, 32, 0.2, 29, 8, v_mix=True), moe(4, 0, 4, 1, 1, 0.9, 40, 3.0)),
    layer(rotary(3, 1, 48, 64, 0.15, 64, 48, base=1000.0), dense(64)),
])
# dense feed-forwards only, head sizes of the matrix-core kernels: the bfloat16 kernels of both mixers
DENSE = model(64, 150, [
    layer(normed(4, 2, 32, 32, 0.2, 24, 10.0, v_mix=True), dense(96)),
    layer(rotary(4, 4, 16, 16, 0.25, 50, 16, v_mix=True), dense(32)),
    layer(normed(2, 1, 48, 80, 0.1, 9, 50.0)),
])

# sizes in no whole eights again, and nothing discrete: dense feed-forwards and routers that choose everything (bfloat16)
ODD_SAFE = model(100, 77, [
    layer(rotary(3, 3, 20, 6, 0.4, 7, 8, base=300.0), moe(3, 1, 4, 2, 2, 1.5, 28, 0.8, shared=(20, 1.2))),
    layer(normed(6, 2, 12, 10, 0.3, 5, 7.0, v_mix=True), dense(28)),
    layer(normed(5, 1, 6, 20, 0.9, 37, 2.5, v_mix=True)),
], eps=1e-3)

CONFIGS = {"odd": ODD, "odd_safe": ODD_SAFE, "general": GENERAL, "all_chosen": ALL_CHOSEN, "dense": DENSE}
PAGE = {"odd": 16, "odd_safe": 16, "general": 16, "all_chosen": 8, "dense": 4}
SEED = {"odd": 14, "odd_safe": 18, "general": 15, "all_chosen": 16, "dense": 17}


def random_weights(cfg: dict, seed: int) -> dict:
    """name -> float32 array for every tensor the configuration needs (shapes asked from the engine's plan, values the
    tests' own): the table N(0, 1), matrices N(0, 0.08), norm weights 1 + N(0, 0.1), biases N(0, 0.1), sinks N(0, 1),
    blend factors in (0.2, 0.8), corrections N(0, 0.05), routers N(0, 0.4)."""
    import sprout_lm_amd as S
    from sprout_lm_amd.registry import build_model_plan
    expected = build_model_plan(S.config_from_dict(cfg)).expected_tensors()
    rng = np.random.default_rng(seed)
    out = {}
    for name in sorted(expected):
        shape = tuple(expected[name].shape)
        last = name.split(".")[-1]
        if name == "embed":
            a = rng.normal(0.0, 1.0, shape)
        elif last in ("norm", "norm1", "norm2"):
            a = 1.0 + rng.normal(0.0, 0.1, shape)
        elif last == "b":
            a = rng.normal(0.0, 0.1, shape)
        elif last == "sink":
            a = rng.normal(0.0, 1.0, shape)
        elif last == "vmix":
            a = rng.uniform(0.2, 0.8, shape)
        elif last == "correction":
            a = rng.normal(0.0, 0.05, shape)
        elif last in ("router", "sg"):
            a = rng.normal(0.0, 0.4, shape)
        else:
            a = rng.normal(0.0, 0.08, shape)
        out[name] = B.bf16_round(np.asarray(a, dtype=np.float32)).reshape(shape)
    return out


def write_folder(folder: str, cfg: dict, weights: dict) -> str:
    from sprout_lm_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      {n: torch.from_numpy(np.ascontiguousarray(a)).reshape(np.shape(a)).to(torch.bfloat16) for n, a in weights.items()})
    return folder


def make_folder(root: str, name: str) -> str:
    folder = os.path.join(root, "bogilix_" + name)
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
            _MODELS[folder] = B.load_folder(folder)
        cfg, w = _MODELS[folder]
        _LOGITS[key] = B.forward(w, cfg, list(tokens), store=B.bf16_round if dtype == "bfloat16" else B.f32)
    return _LOGITS[key]


def tolerance(dtype: str, ref: np.ndarray) -> float:
    """Bound of |engine - plain| on a row of logits: float32 sums against float64 sums, or one-unit flips of the
    bfloat16 roundings that both sides make at the same places."""
    return (2e-5 if dtype == "float32" else 3e-2) * max(1.0, float(np.abs(ref).max()))


def random_tokens(vocab: int, n: int, seed: int) -> list[int]:
    return [int(t) for t in np.random.default_rng(seed).integers(0, vocab, n)]
