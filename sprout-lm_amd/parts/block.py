"""Arrangement of parts in a layer (reference: src/qwen.ts:164-202)."""
from __future__ import annotations

from .base import Block, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    """x += mixer(norm(x)); x += feed_forward(norm(x)).  The residual stream x is float32.  `ffn` (and its norm) may
    be absent: the layer is then its mixer alone."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, mixer_norm, mixer, ffn_norm=None, ffn=None):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        named = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.ffn is not None:
            named.update({"ffn_norm": self.ffn_norm, "ffn": self.ffn})
        return named

    def forward(self, ctx, residual, caches):
        T, H = residual.shape
        cache = caches.get("mixer")
        h = ctx.buffer("normed", (T, H), ctx.act_dtype)
        if not self.mixer.forward_from_residual(ctx, self.mixer_norm, residual, cache):
            self.mixer_norm.forward(ctx, residual, h)
            self.mixer.forward(ctx, h, residual, cache)
        if self.ffn is None:
            return
        if not self.ffn.forward_from_residual(ctx, self.ffn_norm, residual):
            self.ffn_norm.forward(ctx, residual, h)
            self.ffn.forward(ctx, h, residual)


@register_part("block", "parallel")
class ParallelBlock(Block):
    """x += mixer(norm_a(x)) + feed_forward(norm_b(x)): both norms read the same x, so both are taken before
    either part adds into the float32 residual stream.  `ffn` (and its norm) may be absent."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, mixer_norm, mixer, ffn_norm=None, ffn=None):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        named = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.ffn is not None:
            named.update({"ffn_norm": self.ffn_norm, "ffn": self.ffn})
        return named

    def forward(self, ctx, residual, caches):
        T, H = residual.shape
        h = ctx.buffer("normed", (T, H), ctx.act_dtype)
        if self.ffn is None:
            self.mixer_norm.forward(ctx, residual, h)
        else:
            h2 = ctx.buffer("normed_ffn", (T, H), ctx.act_dtype)
            pair = getattr(self.mixer_norm, "forward_pair", None)      # norms that share their statistics take one pass
            if pair is None or not pair(ctx, self.ffn_norm, residual, h, h2):
                self.mixer_norm.forward(ctx, residual, h)
                self.ffn_norm.forward(ctx, residual, h2)
        self.mixer.forward(ctx, h, residual, caches.get("mixer"))
        if self.ffn is not None:
            self.ffn.forward(ctx, h2, residual)
