"""Bogilix as a plan of parts.

Tensor names: `embed`, `final.norm`, `final.norm.b`, `head`; layer i's start with `l<i>.`: `norm1`, `norm1.b`, `norm2`,
`norm2.b`; the mixer's under `mix.` (`q`, `k`, `v`, `o`, biases `q.b` ..., row norms `q.norm`, `k.norm`, `vmix`, `sink`);
the feed-forward's under `mlp.` (`gate`, `up`, `down`, or `e<n>.gate|up|down`, `router`, `correction`,
`shared.gate|up|down`, `shared.sg`).
"""
from __future__ import annotations

from ..config.bogilix import BogilixConfig
from .plan import LayerCall, LayerPlan, ModelPlan, PartPlan

# The design gives no position limit; the engine's bookkeeping wants one.
MAX_POSITIONS = 1 << 22


def _norm(cfg: BogilixConfig, name: str, prefix: str = "") -> PartPlan:
    return PartPlan("norm", "layernorm", {"size": cfg.width, "eps": cfg.eps, "tensor": name, "bias": name + ".b"}, prefix)


def _layer(cfg: BogilixConfig, i: int, first_mixing: int | None) -> LayerPlan:
    entry, base, W = cfg.layers[i], f"l{i}.", cfg.width
    m = entry.mixer
    if m.rot is not None and m.rot[0] > 0:
        position = PartPlan("position", "rotary_neox", {"head_dim": m.dim, "theta": m.rot[1], "rotary_dim": m.rot[0]})
    else:
        position = PartPlan("position", "none", {"head_dim": m.dim})
    normed = entry.kind == "attention_2"
    parts = {
        "mixer_norm": _norm(cfg, "norm1", base),
        "mixer": PartPlan("mixer", "sink_attention", {
            "hidden": W, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
            "position": position, "qkv_bias": normed, "qk_norm": normed, "eps": cfg.eps, "softcap": m.softcap,
            "mask_chunk": m.chunk, "sinks": True,
            "value_mix": None if not m.v_mix else "first" if i == first_mixing else "blend"}, base + "mix."),
    }
    f = entry.mlp
    if f is not None:
        parts["ffn_norm"] = _norm(cfg, "norm2", base)
        if f.kind == "dense":
            parts["ffn"] = PartPlan("feed_forward", "gated_mlp", {"hidden": W, "inner": f.ff, "activation": "silu",
                                                                  "tensors": ("gate", "up", "down")}, base + "mlp.")
        else:
            parts["ffn"] = PartPlan("feed_forward", "routed_experts", {
                "hidden": W, "inner": f.ff, "experts": f.experts, "top": f.top, "router_bias": False,
                "activation": "clamped_swish", "limit": f.limit, "routing": "scored_groups", "identity": f.identity,
                "groups": f.groups, "keep": f.keep, "route_scale": f.scale, "correction": "correction",
                "shared_inner": f.shared[0] if f.shared else None, "shared_limit": f.shared[1] if f.shared else 0.0,
                "shared_activation": "clamped_swish" if f.shared else None,
                "shared_gate": "shared.sg" if f.shared else None}, base + "mlp.")
    return LayerPlan("pre_norm", parts)


def build_bogilix(cfg: BogilixConfig) -> ModelPlan:
    W = cfg.width
    mixing = [i for i, layer in enumerate(cfg.layers) if layer.mixer.v_mix]
    first_mixing = mixing[0] if mixing else None
    return ModelPlan(
        architecture=cfg.architecture, config=cfg, hidden_size=W, vocab_size=cfg.vocab, max_positions=MAX_POSITIONS,
        eos_token_ids=(), embedding=PartPlan("embedding", "token_embedding", {"vocab": cfg.vocab, "hidden": W, "tensor": "embed"}),
        layers=[_layer(cfg, i, first_mixing) for i in range(len(cfg.layers))],
        schedule=[LayerCall(i, i) for i in range(len(cfg.layers))],
        final_norm=_norm(cfg, "final.norm"),
        head=PartPlan("head", "linear_head", {"vocab": cfg.vocab, "hidden": W, "tied": False, "tensor": "head"}))
