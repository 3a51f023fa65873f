"""Configuration of the Megozen decoder: a list of layers, each with a mixer over a cached latent and a
feed-forward of routed experts, on an embedding that adds a hashed-pair (bigram) table."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, ClassVar, Mapping

from .base import ConfigError, ModelConfig, positive_float, positive_int


def _section(raw: Mapping, key: str, where: str, optional: bool = False):
    value = raw.get(key)
    if value is None and optional:
        return None
    if not isinstance(value, Mapping):
        raise ConfigError(f"Invalid Megozen config: {where}{key} must be an object, got {value!r}.")
    return value


def _count(raw: Mapping, key: str, where: str, least: int = 1) -> int:
    value = raw.get(key)
    if isinstance(value, bool) or not isinstance(value, int) or value < least:
        raise ConfigError(f"Invalid Megozen config: {where}{key} must be an integer of at least {least}, got {value!r}.")
    return value


def _number(raw: Mapping, key: str, where: str) -> float:
    value = raw.get(key)
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value) or value <= 0:
        raise ConfigError(f"Invalid Megozen config: {where}{key} must be a positive finite number, got {value!r}.")
    return float(value)


@dataclass(frozen=True)
class RotarySizes:
    dims: int                 # how many numbers of a rotated part turn
    base: float
    scaling: tuple | None     # (factor, original, fast, slow) or None

    @classmethod
    def parse(cls, raw: Mapping, where: str) -> "RotarySizes":
        dims = _count(raw, "dims", where, 0)
        if dims % 2:
            raise ConfigError(f"Invalid Megozen config: {where}dims must be even, got {dims}.")
        scaling = _section(raw, "scaling", where, optional=True)
        if scaling is not None:
            scaling = tuple(_number(scaling, k, where + "scaling.") for k in ("factor", "original", "fast", "slow"))
        return cls(dims, _number(raw, "base", where), scaling)

    def to_dict(self) -> dict:
        out = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        return out

    def scaling_dict(self):
        return None if self.scaling is None else dict(zip(("factor", "original", "fast", "slow"), self.scaling))


@dataclass(frozen=True)
class LatentMixerSizes:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int | None
    rot: RotarySizes

    @classmethod
    def parse(cls, raw: Mapping, where: str) -> "LatentMixerSizes":
        mask = _section(raw, "mask", where, optional=True)
        window = _count(mask, "size", where + "mask.") if mask is not None else None
        rot = RotarySizes.parse(_section(raw, "rot", where), where + "rot.")
        rot_dim = _count(raw, "rot_dim", where, 0)
        if rot.dims > rot_dim:
            raise ConfigError(f"Invalid Megozen config: {where}rot.dims {rot.dims} exceeds rot_dim {rot_dim}.")
        return cls(_count(raw, "heads", where), _count(raw, "dim", where, 0), rot_dim, _count(raw, "vdim", where),
                   _count(raw, "kv_rank", where), _number(raw, "scale", where), window, rot)

    def to_dict(self) -> dict:
        out = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "rot": self.rot.to_dict(),
               "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class ExpertSizes:
    experts: int
    top: int
    inner: int
    shared_inner: int | None

    @classmethod
    def parse(cls, raw: Mapping, where: str) -> "ExpertSizes":
        if raw.get("kind") != "moe":
            raise ConfigError(f"Invalid Megozen config: {where}kind must be 'moe', got {raw.get('kind')!r}.")
        router = _section(raw, "router", where)
        experts, top = _count(router, "experts", where + "router."), _count(router, "top", where + "router.")
        if top > experts:
            raise ConfigError(f"Invalid Megozen config: {where}router.top {top} exceeds the {experts} experts.")
        shared = _section(raw, "shared", where, optional=True)
        return cls(experts, top, _count(_section(raw, "expert", where), "ff", where + "expert."),
                   _count(shared, "ff", where + "shared.") if shared is not None else None)

    def to_dict(self) -> dict:
        out = {"expert": {"ff": self.inner}, "kind": "moe", "router": {"experts": self.experts, "top": self.top}}
        if self.shared_inner is not None:
            out["shared"] = {"ff": self.shared_inner}
        return out


@dataclass(frozen=True)
class MegozenLayer:
    kind: str                       # which mixer
    mixer: LatentMixerSizes
    mlp: ExpertSizes | None
    weights_of: int | None          # the layer whose tensors this one runs with (its cache is its own)

    def to_dict(self) -> dict:
        out = {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None,
               "type": self.kind}
        if self.weights_of is not None:
            out["weights_of"] = self.weights_of
        return out


@dataclass(frozen=True)
class MegozenConfig(ModelConfig):
    """Every size and constant of a Megozen model, as config.json gives them; nothing has a default."""

    architecture: ClassVar[str] = "Megozen"
    mixers: ClassVar[tuple[str, ...]] = ("latent_attention",)

    vocab: int
    width: int
    eps: float
    bigram: tuple | None            # (buckets, mul_prev, mul_cur)
    layers: tuple[MegozenLayer, ...]

    # what the engine asks of every configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "MegozenConfig":
        if not isinstance(raw, Mapping):
            raise ConfigError("Invalid Megozen config: expected a JSON object.")
        if raw.get("architecture") != cls.architecture:
            raise ConfigError(f"Not a Megozen config: architecture is {raw.get('architecture')!r}.")
        vocab, width = positive_int(raw, "vocab"), positive_int(raw, "width")
        eps = positive_float(_section(raw, "norm", ""), "eps")
        embedding = _section(raw, "embedding", "", optional=True) or {}
        bigram = _section(embedding, "bigram", "embedding.", optional=True)
        if bigram is not None:
            bigram = (_count(bigram, "buckets", "embedding.bigram."), _count(bigram, "mul_prev", "embedding.bigram.", 0),
                      _count(bigram, "mul_cur", "embedding.bigram.", 0))
        entries = raw.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("Invalid Megozen config: layers must be a non-empty list.")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]."
            if not isinstance(entry, Mapping):
                raise ConfigError(f"Invalid Megozen config: layers[{i}] must be an object.")
            kind = entry.get("type")
            if kind not in cls.mixers:
                raise ConfigError(f"Invalid Megozen config: {where}type {kind!r} is no mixer of this design {cls.mixers}.")
            mixer = LatentMixerSizes.parse(_section(entry, "mixer", where), where + "mixer.")
            mlp = _section(entry, "mlp", where, optional=True)
            source = entry.get("weights_of")
            if source is not None and (isinstance(source, bool) or not isinstance(source, int)
                                       or not 0 <= source < len(entries) or source == i):
                raise ConfigError(f"Invalid Megozen config: {where}weights_of {source!r} names no other layer.")
            layers.append(MegozenLayer(kind, mixer, ExpertSizes.parse(mlp, where + "mlp.") if mlp is not None else None,
                                       source))
        config = cls(vocab, width, eps, bigram, tuple(layers))
        for i in range(len(layers)):
            config.source_of(i)
        return config

    def source_of(self, i: int) -> int:
        """The layer whose tensors layer i runs with (itself, unless it names another, which may name a third)."""
        seen = {i}
        while self.layers[i].weights_of is not None:
            i = self.layers[i].weights_of
            if i in seen:
                raise ConfigError("Invalid Megozen config: weights_of runs in a circle.")
            seen.add(i)
        return i

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "layers": [layer.to_dict() for layer in self.layers],
               "norm": {"eps": self.eps}, "vocab": self.vocab, "width": self.width}
        if self.bigram is not None:
            out["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), self.bigram))}
        return out
