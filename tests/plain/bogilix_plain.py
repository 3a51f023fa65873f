"""Plain Bogilix forward pass: whole sequence, no cache, float64 arithmetic, one function per mechanism.

Shares no code with the engine.  `store` is an optional rounding function applied wherever the bfloat16 engine
keeps a tensor in bfloat16 (normed activations, projection outputs, cached keys and values, the attention output,
gated products); with the default (float32 rounding) everything is float32 storage over float64 sums.

Notation.  x: the residual stream [tokens, width].  A layer is x <- x + mixer(ln1(x)), then x <- x + ff(ln2(x)),
with layer norms that carry a weight and a bias.  Two mixers, both grouped-query attention inside blocks of
`mask.size` positions (a query sees the earlier keys of its own block only), with one learned logit per head in the
softmax's denominator that has no value, and with the values of every flagged layer after the first blended with the
first flagged layer's values of the same token:
  "attention"    no biases, the first rot.dims numbers of every head turned by position ("halves" pairing);
  "attention_2"  biases on q, k, v, an RMS norm over the whole q row and the whole k row, no positions at all,
                 scores squashed to (-cap, cap) by a tanh.
Feed-forwards: a dense gated one (SiLU), or routed experts (softmax over all router outputs, a correction added
for the choice only, the choice limited to the best groups of neighbouring experts, trailing identity experts that
return their input, a shared expert behind a sigmoid gate of one number per token).
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


# ---------------------------------------------------------------------------------------------- small pieces
def sigmoid(z):
    z = np.asarray(z, dtype=np.float64)
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    z = np.asarray(z, dtype=np.float64)
    return z * sigmoid(z)


def linear(x, w, b=None):
    y = np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T
    return y if b is None else y + np.asarray(b, dtype=np.float64)


def layer_norm(x, weight, bias, eps):
    """(x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b."""
    x = np.asarray(x, dtype=np.float64)
    d = x - x.mean(axis=-1, keepdims=True)
    return d / np.sqrt((d * d).mean(axis=-1, keepdims=True) + eps) * np.asarray(weight, dtype=np.float64) + np.asarray(bias, dtype=np.float64)


def rms_norm(x, weight, eps):
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * np.asarray(weight, dtype=np.float64)


def turn_halves(x, positions, dims: int, base: float):
    """x [tokens, heads, size]: number i of a head turns with number i + dims/2 by positions * base^(-2i/dims);
    numbers from `dims` on stay."""
    x = np.array(x, dtype=np.float64)
    half = dims // 2
    if half == 0:
        return x
    freq = float(base) ** (-2.0 * np.arange(half, dtype=np.float64) / dims)
    angle = np.asarray(positions, dtype=np.float64)[:, None, None] * freq[None, None, :]
    c, s = np.cos(angle), np.sin(angle)
    a, b = x[..., :half].copy(), x[..., half:dims].copy()
    x[..., :half] = a * c - b * s
    x[..., half:dims] = b * c + a * s
    return x


def block_mask(n: int, size: int):
    """[query, key]: key j <= query i and both in the same block of `size` positions counted from 0."""
    i = np.arange(n)[:, None]
    j = np.arange(n)[None, :]
    return (j <= i) & (i // size == j // size)


def softmax_with_sink(scores, allowed, sink):
    """Weights of the allowed keys where the denominator also holds exp(sink), a term without a key."""
    s = np.where(allowed, scores, -np.inf)
    top = np.maximum(s.max(axis=-1, keepdims=True), sink)
    e = np.exp(s - top)
    return e / (e.sum(axis=-1, keepdims=True) + np.exp(sink - top))


def attend(q, k, v, heads: int, kv_heads: int, scale: float, size: int, sinks, cap=None, store=f32):
    """q [T, heads, dim], k [T, kv_heads, dim], v [T, kv_heads, vdim] -> [T, heads * vdim]."""
    T = q.shape[0]
    per = heads // kv_heads
    allowed = block_mask(T, size)
    out = np.zeros((T, heads, v.shape[2]))
    for h in range(heads):
        g = h // per
        scores = (q[:, h] @ k[:, g].T) * scale
        if cap is not None:
            scores = cap * np.tanh(scores / cap)
        out[:, h] = softmax_with_sink(scores, allowed, float(sinks[h])) @ v[:, g]
    return store(out.reshape(T, -1))


def blend_values(v, first, lam):
    """(1 - lam) v + lam first."""
    return (1.0 - float(lam)) * v + float(lam) * first


# ---------------------------------------------------------------------------------------------- mixers
def mixer_rotary(w, pre, m, h, positions, shared, store=f32):
    """Mixer "attention": no biases, the first rot.dims numbers of every head turn."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = store(linear(h, w[pre + "q"])).reshape(T, H, D)
    k = store(linear(h, w[pre + "k"])).reshape(T, G, D)
    v = store(linear(h, w[pre + "v"])).reshape(T, G, V)
    rot = m.get("rot")
    if rot:
        q = store(turn_halves(q, positions, rot["dims"], rot["base"]))
        k = store(turn_halves(k, positions, rot["dims"], rot["base"]))
    v = _values(w, pre, m, v, shared, store)
    a = attend(q, k, v, H, G, m["scale"], m["mask"]["size"], w[pre + "sink"], None, store)
    return linear(a, w[pre + "o"])


def mixer_normed(w, pre, m, h, eps, shared, store=f32):
    """Mixer "attention_2": biases, RMS norm over the whole q row and the whole k row, no positions, capped scores."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = store(linear(h, w[pre + "q"], w[pre + "q.b"]))
    k = store(linear(h, w[pre + "k"], w[pre + "k.b"]))
    v = store(linear(h, w[pre + "v"], w[pre + "v.b"])).reshape(T, G, V)
    q = store(rms_norm(q, w[pre + "q.norm"], eps)).reshape(T, H, D)
    k = store(rms_norm(k, w[pre + "k.norm"], eps)).reshape(T, G, D)
    v = _values(w, pre, m, v, shared, store)
    a = attend(q, k, v, H, G, m["scale"], m["mask"]["size"], w[pre + "sink"], m["softcap"], store)
    return linear(a, w[pre + "o"])


def _values(w, pre, m, v, shared, store):
    if not m.get("v_mix"):
        return v
    if "first" not in shared:
        shared["first"] = v
        return v
    return store(blend_values(v, shared["first"].reshape(v.shape), np.asarray(w[pre + "vmix"]).reshape(())))


# ---------------------------------------------------------------------------------------------- feed-forwards
def dense_ff(w, pre, h, store=f32):
    act = store(silu(store(linear(h, w[pre + "gate"]))) * store(linear(h, w[pre + "up"])))
    return linear(act, w[pre + "down"])


def expert(w, pre, h, limit: float, store=f32):
    """down((g * sigmoid(1.702 g)) * (u + 1)), g = min(gate h, limit), u = clamp(up h, -limit, limit)."""
    g = np.minimum(store(linear(h, w[pre + "gate"])), limit)
    u = np.clip(store(linear(h, w[pre + "up"])), -limit, limit)
    return linear(store(g * sigmoid(1.702 * g) * (u + 1.0)), w[pre + "down"])


def route(z, correction, top: int, groups: int, keep: int, scale: float):
    """z [T, n] router outputs (real experts then identity experts) -> (chosen [T, top], weights [T, top])."""
    z = np.asarray(z, dtype=np.float64)
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    s = e / e.sum(axis=-1, keepdims=True)
    choice = s + np.asarray(correction, dtype=np.float64)
    T, n = z.shape
    per = n // groups
    best = choice.reshape(T, groups, per).max(axis=-1)
    chosen = np.zeros((T, top), dtype=np.int64)
    weights = np.zeros((T, top))
    for t in range(T):
        kept = np.argsort(-best[t], kind="stable")[:keep]
        open_ = np.full(n, -np.inf)
        for g in kept:
            open_[g * per:(g + 1) * per] = choice[t, g * per:(g + 1) * per]
        chosen[t] = np.argsort(-open_, kind="stable")[:top]
        weights[t] = s[t, chosen[t]] * scale
    return chosen, weights


def routed_ff(w, pre, f, h, store=f32, router_input=None):
    r = f["router"]
    E, I = r["experts"], r.get("identity", 0)
    hr = h if router_input is None else router_input
    chosen, weights = route(linear(hr, w[pre + "router"]), w[pre + "correction"], r["top"], r["groups"]["count"],
                            r["groups"]["keep"], r["scale"])
    out = np.zeros((h.shape[0], w[pre + "router"].shape[1]))
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t], weights[t]):
            if e >= E:
                out[t] += a * np.asarray(h[t], dtype=np.float64)
            else:
                out[t] += a * expert(w, f"{pre}e{e}.", h[t:t + 1], f["expert"]["limit"], store)[0]
    if f.get("shared"):
        gate = sigmoid(linear(hr, w[pre + "shared.sg"]))
        out += gate * expert(w, pre + "shared.", h, f["shared"]["limit"], store)
    return out


# ---------------------------------------------------------------------------------------------- the model
def forward(w, cfg, tokens, store=f32, rows=None, streams=None):
    """Logits [len(rows) or T, vocab] of the whole sequence.  `streams`: a list that receives x after every layer."""
    eps = cfg["norm"]["eps"]
    x = np.asarray(w["embed"], dtype=np.float64)[np.asarray(tokens)]
    positions = np.arange(len(tokens))
    shared = {}
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = store(layer_norm(x, w[pre + "norm1"], w[pre + "norm1.b"], eps))
        if layer["type"] == "attention":
            x = x + mixer_rotary(w, pre + "mix.", layer["mixer"], h, positions, shared, store)
        elif layer["type"] == "attention_2":
            x = x + mixer_normed(w, pre + "mix.", layer["mixer"], h, eps, shared, store)
        else:
            raise ValueError(layer["type"])
        f = layer.get("mlp")
        if f is not None:
            h = store(layer_norm(x, w[pre + "norm2"], w[pre + "norm2.b"], eps))
            x = x + (dense_ff(w, pre + "mlp.", h, store) if f["kind"] == "dense" else routed_ff(w, pre + "mlp.", f, h, store))
        if streams is not None:
            streams.append(x.copy())
    if rows is not None:
        x = x[np.asarray(rows)]
    x = store(layer_norm(x, w["final.norm"], w["final.norm.b"], eps))
    return linear(x, w["head"]).astype(np.float32)


def forward_logits(w, cfg, tokens, store=f32, rows=None):
    return forward(w, cfg, tokens, store=store, rows=rows)
