"""Plain Megozen forward pass: whole sequence, no cache, float64 arithmetic, one function per mechanism.

Shares no code with the engine.  `store` is an optional rounding function applied wherever the bfloat16 engine
keeps a tensor in bfloat16 (normed activations, projection outputs, the cached latent and rotated key part, the
attention output, expert activations); with the default (float32 rounding) everything is float32 storage over
float64 sums.

Notation.  x: the residual stream [tokens, width].  A layer is x <- x + mixer(ln1(x)) + ff(ln2(x)), both norms
of the same x.  The mixer is attention over a latent: per token a latent c (kv_rank numbers, RMS-normed) and one
rotated key part r (rot_dim numbers) shared by all heads are what later tokens read; head h scores a key as
(q_h[:dim] . (U_k,h c) + rot(q_h[dim:]) . rot(r)) * scale and sums values U_v,h c.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np


def f32(x):
    return np.asarray(x, dtype=np.float64).astype(np.float32)


def bf16_round(x):
    a = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    bits = a.view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return rounded.astype(np.uint32).view(np.float32).reshape(a.shape)


def read_safetensors(path: str) -> dict:
    """name -> float64 (or integer) array: 8 bytes of header length, the JSON header, then the data."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        lo, hi = meta["data_offsets"]
        raw = data[lo:hi]
        if meta["dtype"] == "BF16":
            a = (np.frombuffer(raw, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif meta["dtype"] == "F32":
            a = np.frombuffer(raw, dtype=np.float32).astype(np.float64)
        elif meta["dtype"] == "I32":
            a = np.frombuffer(raw, dtype=np.int32)
        else:
            raise ValueError(f"{name}: dtype {meta['dtype']}")
        out[name] = a.reshape(meta["shape"])
    return out


def load_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


# ---------------------------------------------------------------------------------------------- mechanisms
def gelu_tanh(z):
    z = np.asarray(z, dtype=np.float64)
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    z = np.asarray(z, dtype=np.float64)
    return z / (1.0 + np.exp(-z))


def linear(x, w):
    return np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T


def layer_norm(x, weight, eps):
    """(x - mean) / sqrt(mean((x - mean)^2) + eps) * w, no bias."""
    x = np.asarray(x, dtype=np.float64)
    d = x - x.mean(axis=-1, keepdims=True)
    return d / np.sqrt((d * d).mean(axis=-1, keepdims=True) + eps) * np.asarray(weight, dtype=np.float64)


def rms_norm(x, weight, eps):
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * np.asarray(weight, dtype=np.float64)


def bigram_rows(tokens, buckets: int, mul_prev: int, mul_cur: int):
    """Row of the bigram table for every token: a hash of (previous, current); the first token takes the last row."""
    rows = [buckets]
    for prev, cur in zip(tokens[:-1], tokens[1:]):
        rows.append((prev * mul_prev + cur * mul_cur) % buckets)
    return np.asarray(rows[:len(tokens)], dtype=np.int64)


def embed(w, cfg, tokens):
    x = np.asarray(w["embed"], dtype=np.float64)[np.asarray(tokens)]
    big = (cfg.get("embedding") or {}).get("bigram")
    if big:
        x = x + np.asarray(w["bigram"], dtype=np.float64)[bigram_rows(list(tokens), big["buckets"], big["mul_prev"], big["mul_cur"])]
    return x


def yarn_frequencies(rot: dict):
    """(frequency of every pair, factor on cosines and sines)."""
    dims, base = rot["dims"], float(rot["base"])
    i = np.arange(dims // 2, dtype=np.float64)
    freq = base ** (-2.0 * i / dims)
    scaling = rot.get("scaling")
    if not scaling:
        return freq, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return freq / factor * ramp + freq * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x, positions, rot: dict, angle_dtype=np.float64):
    """x [..., tokens, n]: the first rot.dims numbers turn, (2i, 2i + 1) together; the rest pass."""
    x = np.asarray(x, dtype=np.float64)
    dims = rot["dims"]
    freq, magnitude = yarn_frequencies(rot)
    angle = (np.asarray(positions, dtype=angle_dtype)[:, None] * freq.astype(angle_dtype)[None, :]).astype(np.float64)
    cos, sin = np.cos(angle) * magnitude, np.sin(angle) * magnitude
    out = x.copy()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def window_mask(n: int, window):
    """[query, key]: key j is seen from i if 0 <= i - j < window (every earlier key without a window)."""
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    seen = j <= i
    if window:
        seen &= (i - j) < window
    return seen


def softmax_rows(scores, seen):
    s = np.where(seen, scores, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    return e / e.sum(axis=-1, keepdims=True)


def latent_attention(w, prefix: str, m: dict, h, positions, eps, store=f32, angle_dtype=np.float64):
    """The mixer on normed input h [tokens, width]; `m` is the layer's `mixer` entry."""
    H, dim, rd, vd, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    n = h.shape[0]
    q = store(linear(h, w[prefix + "q"])).reshape(n, H, dim + rd).astype(np.float64)
    dkv = store(linear(h, w[prefix + "dkv"])).astype(np.float64)
    c = store(rms_norm(dkv[:, :rank], w[prefix + "dkv.norm"], eps)).astype(np.float64)
    k_rot = store(rotate_interleaved(dkv[:, rank:], positions, m["rot"], angle_dtype)).astype(np.float64)
    q_rot = store(rotate_interleaved(q[:, :, dim:].transpose(1, 0, 2), positions, m["rot"], angle_dtype)).astype(np.float64)
    k_un = linear(c, w[prefix + "uk"]).reshape(n, H, dim)
    v = linear(c, w[prefix + "uv"]).reshape(n, H, vd)
    seen = window_mask(n, (m.get("mask") or {}).get("size"))
    gate = 1.0 / (1.0 + np.exp(-store(linear(h, w[prefix + "g"])).astype(np.float64)))
    out = np.zeros((n, H, vd))
    for head in range(H):
        scores = (q[:, head, :dim] @ k_un[:, head].T + q_rot[head] @ k_rot.T) * m["scale"]
        out[:, head] = softmax_rows(scores, seen) @ v[:, head]
    out = store(out * gate[:, :, None]).astype(np.float64)
    return linear(out.reshape(n, H * vd), w[prefix + "o"])


def gated_expert(w, prefix: str, h):
    return linear(silu(linear(h, w[prefix + "gate"])) * linear(h, w[prefix + "up"]), w[prefix + "down"])


def route(logits, top: int):
    """(chosen experts [tokens, top], their weights): the `top` largest logits, softmax over those alone."""
    order = np.argsort(-logits, axis=-1, kind="stable")[:, :top]
    chosen = np.take_along_axis(logits, order, axis=-1)
    e = np.exp(chosen - chosen.max(axis=-1, keepdims=True))
    return order, e / e.sum(axis=-1, keepdims=True)


def moe(w, prefix: str, mlp: dict, h):
    """Routed experts plus the shared one, on normed input h.  Also returns the gap between the last chosen and
    the first refused router logit of every token (a token on that edge may go either way under rounding)."""
    experts, top = mlp["router"]["experts"], mlp["router"]["top"]
    logits = linear(h, w[prefix + "router"]) + np.asarray(w[prefix + "router.b"], dtype=np.float64)
    chosen, weight = route(logits, top)
    ranked = -np.sort(-logits, axis=-1)
    gap = ranked[:, top - 1] - ranked[:, top] if experts > top else np.full(len(h), np.inf)
    out = np.zeros((h.shape[0], w[prefix + "e0.down"].shape[0]))
    for e in range(experts):
        rows, slot = np.nonzero(chosen == e)
        if len(rows):
            out[rows] += weight[rows, slot][:, None] * gated_expert(w, f"{prefix}e{e}.", h[rows])
    if mlp.get("shared"):
        out += gated_expert(w, prefix + "shared.", h)
    return out, gap


def run_order(cfg):
    """(layer whose tensors run, the entry) for every layer of the list."""
    def owner(i):
        while cfg["layers"][i].get("weights_of") is not None:      # a layer may name one that names a third
            i = cfg["layers"][i]["weights_of"]
        return i
    return [(owner(i), entry) for i, entry in enumerate(cfg["layers"])]


def forward(w, cfg, tokens, store=f32, rows=None, angle_dtype=np.float64, trace=None):
    """Logits [len(rows) or tokens, vocab] in float64.  `trace`: a list that receives the residual stream after
    every layer run, and (as its last element) the smallest router gap seen."""
    eps = cfg["norm"]["eps"]
    positions = np.arange(len(tokens))
    x = embed(w, cfg, tokens)
    smallest = np.inf
    for source, entry in run_order(cfg):
        p = f"l{source}."
        if entry["type"] != "latent_attention":
            raise ValueError(entry["type"])
        h1 = store(layer_norm(x, w[p + "norm1"], eps)).astype(np.float64)
        add = latent_attention(w, p + "mix.", entry["mixer"], h1, positions, eps, store, angle_dtype)
        if entry.get("mlp"):
            h2 = store(layer_norm(x, w[p + "norm2"], eps)).astype(np.float64)
            ff, gap = moe(w, p + "mlp.", entry["mlp"], h2)
            smallest = min(smallest, float(gap.min()))
            add = add + ff
        x = f32(x + add).astype(np.float64)
        if trace is not None:
            trace.append(x.copy())
    if trace is not None:
        trace.append(smallest)
    if rows is not None:
        x = x[np.asarray(rows)]
    return linear(store(layer_norm(x, w["final.norm"], eps)), w["head"])
