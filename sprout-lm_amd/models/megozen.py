"""Megozen as a plan of parts.

Tensor names: `embed`, `bigram`, `final.norm`, `head`; layer i's start with `l<i>.`: `norm1`, `norm2`, the mixer's
under `mix.` and the feed-forward's under `mlp.` (`e<n>.gate|up|down`, `router`, `router.b`, `shared.gate|up|down`).
A layer that names another under `weights_of` runs with that layer's parts and a cache of its own: in the plan it
is a second call of the same layer with another cache slot.
"""
from __future__ import annotations

from ..config.megozen import MegozenConfig
from .plan import LayerCall, LayerPlan, ModelPlan, PartPlan

# The design gives no position limit; the engine's bookkeeping wants one.
MAX_POSITIONS = 1 << 22


def _layer(cfg: MegozenConfig, i: int) -> LayerPlan:
    entry, base, W = cfg.layers[i], f"l{i}.", cfg.width
    m = entry.mixer
    position = PartPlan("position", "rotary_interleaved", {"rotary_dim": m.rot.dims, "theta": m.rot.base,
                                                           "scaling": m.rot.scaling_dict()})
    parts = {
        "mixer_norm": PartPlan("norm", "layernorm", {"size": W, "eps": cfg.eps, "tensor": "norm1"}, base),
        "mixer": PartPlan("mixer", "latent_attention", {
            "hidden": W, "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
            "scale": m.scale, "eps": cfg.eps, "position": position, "window": m.window, "gated": True}, base + "mix."),
    }
    if entry.mlp is not None:
        f = entry.mlp
        parts["ffn_norm"] = PartPlan("norm", "layernorm", {"size": W, "eps": cfg.eps, "tensor": "norm2"}, base)
        parts["ffn"] = PartPlan("feed_forward", "routed_experts", {
            "hidden": W, "inner": f.inner, "experts": f.experts, "top": f.top, "shared_inner": f.shared_inner,
            "router_bias": True, "activation": "silu"}, base + "mlp.")
    return LayerPlan("parallel", parts)


def build_megozen(cfg: MegozenConfig) -> ModelPlan:
    W = cfg.width
    owners = sorted({cfg.source_of(i) for i in range(len(cfg.layers))})
    index = {layer: n for n, layer in enumerate(owners)}
    schedule = [LayerCall(index[cfg.source_of(i)], i) for i in range(len(cfg.layers))]
    if cfg.bigram is not None:
        buckets, mul_prev, mul_cur = cfg.bigram
        embedding = PartPlan("embedding", "bigram_embedding", {"vocab": cfg.vocab, "hidden": W, "buckets": buckets,
                                                               "mul_prev": mul_prev, "mul_cur": mul_cur,
                                                               "tensors": ("embed", "bigram")})
        embedding_slot = len(schedule)
    else:
        embedding = PartPlan("embedding", "token_embedding", {"vocab": cfg.vocab, "hidden": W, "tensor": "embed"})
        embedding_slot = None
    return ModelPlan(
        architecture=cfg.architecture, config=cfg, hidden_size=W, vocab_size=cfg.vocab, max_positions=MAX_POSITIONS,
        eos_token_ids=(), embedding=embedding, layers=[_layer(cfg, i) for i in owners], schedule=schedule,
        final_norm=PartPlan("norm", "layernorm", {"size": W, "eps": cfg.eps, "tensor": "final.norm"}),
        head=PartPlan("head", "linear_head", {"vocab": cfg.vocab, "hidden": W, "tied": False, "tensor": "head"}),
        embedding_slot=embedding_slot)
