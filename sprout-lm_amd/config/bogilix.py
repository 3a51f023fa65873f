"""Configuration of the Bogilix decoder: a list of layers, each with one of two attention mixers and a dense or routed
feed-forward (or none), between layer norms with bias."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, ClassVar, Mapping

from .base import ConfigError, ModelConfig, positive_float, positive_int

_WHAT = "Invalid Bogilix config: "


def _section(raw: Mapping, key: str, where: str, optional: bool = False):
    value = raw.get(key)
    if value is None and optional:
        return None
    if not isinstance(value, Mapping):
        raise ConfigError(f"{_WHAT}{where}{key} must be an object, got {value!r}.")
    return value


def _count(raw: Mapping, key: str, where: str, least: int = 1) -> int:
    value = raw.get(key)
    if isinstance(value, bool) or not isinstance(value, int) or value < least:
        raise ConfigError(f"{_WHAT}{where}{key} must be an integer of at least {least}, got {value!r}.")
    return value


def _number(raw: Mapping, key: str, where: str) -> float:
    value = raw.get(key)
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value) or value <= 0:
        raise ConfigError(f"{_WHAT}{where}{key} must be a positive finite number, got {value!r}.")
    return float(value)


@dataclass(frozen=True)
class AttentionSizes:
    """Sizes and constants of a mixer.  `rot`: (dims, base) of the rotation, or None where nothing turns; `softcap`:
    None where scores are not capped; `chunk`: positions in a block of the mask."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int
    v_mix: bool
    rot: tuple | None
    softcap: float | None

    @classmethod
    def parse(cls, raw: Mapping, where: str, kind: str) -> "AttentionSizes":
        heads, kv_heads = _count(raw, "heads", where), _count(raw, "kv_heads", where)
        if heads % kv_heads:
            raise ConfigError(f"{_WHAT}{where}heads {heads} are no whole multiple of kv_heads {kv_heads}.")
        dim = _count(raw, "dim", where)
        rot = softcap = None
        if kind == "attention":
            section = _section(raw, "rot", where)
            dims = _count(section, "dims", where + "rot.", 0)
            if dims % 2 or dims > dim:
                raise ConfigError(f"{_WHAT}{where}rot.dims must be even and at most dim {dim}, got {dims}.")
            rot = (dims, _number(section, "base", where + "rot."))
        else:
            softcap = _number(raw, "softcap", where)
        v_mix = raw.get("v_mix", False)
        if not isinstance(v_mix, bool):
            raise ConfigError(f"{_WHAT}{where}v_mix must be true or false, got {v_mix!r}.")
        return cls(heads, kv_heads, dim, _count(raw, "vdim", where), _number(raw, "scale", where),
                   _count(_section(raw, "mask", where), "size", where + "mask."), v_mix, rot, softcap)

    def to_dict(self) -> dict:
        out = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "mask": {"size": self.chunk},
               "scale": self.scale, "v_mix": self.v_mix, "vdim": self.vdim}
        if self.rot is not None:
            out["rot"] = {"base": self.rot[1], "dims": self.rot[0]}
        if self.softcap is not None:
            out["softcap"] = self.softcap
        return out


@dataclass(frozen=True)
class FeedForwardSizes:
    """kind "dense": `ff`.  kind "moe": experts of `ff` with `limit`; the router's `experts`, `identity`, `top`, `groups`,
    `keep`, `scale`; the shared expert's (ff, limit) or None."""

    kind: str
    ff: int
    limit: float = 0.0
    experts: int = 0
    identity: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1
    scale: float = 1.0
    shared: tuple | None = None

    @classmethod
    def parse(cls, raw: Mapping, where: str) -> "FeedForwardSizes":
        kind = raw.get("kind")
        if kind == "dense":
            return cls("dense", _count(raw, "ff", where))
        if kind != "moe":
            raise ConfigError(f"{_WHAT}{where}kind must be 'dense' or 'moe', got {kind!r}.")
        expert, router = _section(raw, "expert", where), _section(raw, "router", where)
        # a router without identity experts or without groups may leave those keys out: no experts of that kind, one group
        groups = _section(router, "groups", where + "router.", optional=True)
        experts = _count(router, "experts", where + "router.")
        identity = _count(router, "identity", where + "router.", 0) if router.get("identity") is not None else 0
        top = _count(router, "top", where + "router.")
        count, keep = (1, 1) if groups is None else (_count(groups, "count", where + "router.groups."),
                                                     _count(groups, "keep", where + "router.groups."))
        outputs = experts + identity
        if outputs % count or keep > count or top > keep * (outputs // count):
            raise ConfigError(f"{_WHAT}{where}router: {outputs} outputs do not form {count} equal groups of which {keep} "
                              f"hold {top} choices.")
        shared = _section(raw, "shared", where, optional=True)
        return cls("moe", _count(expert, "ff", where + "expert."), _number(expert, "limit", where + "expert."), experts,
                   identity, top, count, keep, _number(router, "scale", where + "router."),
                   (_count(shared, "ff", where + "shared."), _number(shared, "limit", where + "shared.")) if shared is not None else None)

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        out = {"expert": {"ff": self.ff, "limit": self.limit}, "kind": "moe",
               "router": {"experts": self.experts, "groups": {"count": self.groups, "keep": self.keep},
                          "identity": self.identity, "scale": self.scale, "top": self.top}}
        if self.shared is not None:
            out["shared"] = {"ff": self.shared[0], "limit": self.shared[1]}
        return out


@dataclass(frozen=True)
class BogilixLayer:
    kind: str                       # "attention" or "attention_2"
    mixer: AttentionSizes
    mlp: FeedForwardSizes | None

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None, "type": self.kind}


@dataclass(frozen=True)
class BogilixConfig(ModelConfig):
    """Every size and constant of a Bogilix model, as config.json gives them; nothing has a default."""

    architecture: ClassVar[str] = "Bogilix"
    mixers: ClassVar[tuple[str, ...]] = ("attention", "attention_2")

    vocab: int
    width: int
    eps: float
    layers: tuple[BogilixLayer, ...]

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "BogilixConfig":
        if not isinstance(raw, Mapping):
            raise ConfigError(_WHAT + "expected a JSON object.")
        if raw.get("architecture") != cls.architecture:
            raise ConfigError(f"Not a Bogilix config: architecture is {raw.get('architecture')!r}.")
        vocab, width = positive_int(raw, "vocab"), positive_int(raw, "width")
        eps = positive_float(_section(raw, "norm", ""), "eps")
        entries = raw.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError(_WHAT + "layers must be a non-empty list.")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]."
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{_WHAT}layers[{i}] must be an object.")
            kind = entry.get("type")
            if kind not in cls.mixers:
                raise ConfigError(f"{_WHAT}{where}type {kind!r} is no mixer of this design {cls.mixers}.")
            mixer = AttentionSizes.parse(_section(entry, "mixer", where), where + "mixer.", kind)
            mlp = _section(entry, "mlp", where, optional=True)
            layers.append(BogilixLayer(kind, mixer, FeedForwardSizes.parse(mlp, where + "mlp.") if mlp is not None else None))
        mixing = [layer.mixer for layer in layers if layer.mixer.v_mix]
        if any(m.kv_heads * m.vdim != mixing[0].kv_heads * mixing[0].vdim for m in mixing):
            raise ConfigError(_WHAT + "layers that blend their values with the first such layer's must have as many value numbers a token.")
        return cls(vocab, width, eps, tuple(layers))

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "layers": [layer.to_dict() for layer in self.layers],
                "norm": {"eps": self.eps}, "vocab": self.vocab, "width": self.width}
