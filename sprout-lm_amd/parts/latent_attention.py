"""Attention over a cached latent: per token one low-rank latent and one rotated key part serve every head."""
from __future__ import annotations

import torch

from .. import ops
from ..cache.spec import PagedKVSpec
from ..config.base import ConfigError
from ..weights.loader import TensorSpec
from .base import Mixer, register_part


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    """Head h scores key j as (q_h[:dim] . (U_k,h c_j) + turn(q_h[dim:]) . turn(r_j)) * scale and sums values
    U_v,h c_j, where c_j (kv_rank numbers, RMS-normed) and r_j (rot_dim numbers) come from one down projection of
    token j; the head's output is multiplied by sigmoid(gate_h) where `gated`, and W_o mixes the heads.

    Only c and turn(r) are cached, and attention runs on them directly: since q . (U_k c) = (U_k^T q) . c, the
    queries are carried into the latent's space by a per-head product, the attention kernels see ONE key/value
    head of width kv_rank + rot_dim shared by all query heads (key [c, turn(r)], value c in the same width), and a
    second per-head product with U_v (and the gate) brings the weighted latents to value size.  A decoded token
    reads kv_rank + rot_dim numbers per key instead of heads * (dim + rot_dim + vdim).

    hidden, heads, dim, rot_dim, vdim, kv_rank: sizes.  scale: the factor on q . k, used as given.  window: None,
    or how many of the latest keys (itself included) a query sees.  position: a PositionEncoding whose `freq`
    (float64 table), `rotary_dim` (how many of the rot_dim numbers turn) and `magnitude` the turning kernel takes;
    neighbours (2i, 2i + 1) turn together.  eps: of the latent's RMS norm.  `tensors`: local names of the query,
    down, latent-norm, key-up, value-up, gate and output tensors.
    """

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, scale: float, eps: float,
                 position, window: int | None = None, gated: bool = True, page_tokens: int | None = None,
                 tensors: tuple = ("q", "dkv", "dkv.norm", "uk", "uv", "g", "o")):
        if min(hidden, heads, dim, vdim, kv_rank) <= 0 or rot_dim < 0:
            raise ConfigError(f"Latent attention needs positive sizes, got heads={heads} dim={dim} rot_dim={rot_dim} "
                              f"vdim={vdim} kv_rank={kv_rank}.")
        if getattr(position, "pairing", None) != "interleaved" and getattr(position, "rotary_dim", 0):
            raise ConfigError("Latent attention turns neighbouring numbers; its position encoding must pair them so.")
        if getattr(position, "rotary_dim", 0) > rot_dim:
            raise ConfigError(f"{position.rotary_dim} numbers cannot turn in a rotated part of {rot_dim}.")
        try:      # one key/value head of width kv_rank + rot_dim under all query heads
            ops.check_attention_sizes(heads, 1, kv_rank + rot_dim)
        except ops.KernelError as error:
            raise ConfigError(str(error)) from None
        self.hidden, self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank = hidden, heads, dim, rot_dim, vdim, kv_rank
        self.scale, self.eps, self.position, self.window, self.gated = float(scale), float(eps), position, window, gated
        self.page_tokens = page_tokens
        self.names = tuple(tensors)
        self.key_width = kv_rank + rot_dim

    # ------------------------------------------------------------------ what it keeps and costs
    def cache_spec(self):
        return PagedKVSpec(1, self.key_width, self.window, self.page_tokens)

    def cache_elements_per_token(self) -> int:
        return 2 * self.key_width

    def flops(self, tokens: int, pairs: int = 0) -> float:
        H = self.heads
        rows_in = H * (self.dim + self.rot_dim) + self.key_width + (H if self.gated else 0)
        products = rows_in * self.hidden + H * self.dim * self.kv_rank + H * self.kv_rank * self.vdim + H * self.vdim * self.hidden
        return 2.0 * tokens * products + 4.0 * H * self.key_width * pairs

    def tensors(self):
        q, dkv, norm, uk, uv, g, o = self.names
        H = self.heads
        out = {q: TensorSpec((H * (self.dim + self.rot_dim), self.hidden)),
               dkv: TensorSpec((self.key_width, self.hidden)),
               norm: TensorSpec((self.kv_rank,), "vector", "one_plus_normal"),
               uk: TensorSpec((H * self.dim, self.kv_rank)),
               uv: TensorSpec((H * self.vdim, self.kv_rank)),
               o: TensorSpec((self.hidden, H * self.vdim))}
        if self.gated:
            out[g] = TensorSpec((H, self.hidden))
        return out

    def bind(self, tensors):
        q, dkv, norm, uk, uv, g, o = self.names
        H = self.heads
        # one product for everything that reads the mixer's input: queries, latent + rotated key part, gates
        # (rows of zeros behind them bring a row of results to a multiple of 8 numbers: every token's row, and with
        # head sizes in eights every head's part of it, then starts at a multiple of 16 bytes for the per-head products)
        stacked = [tensors[q], tensors[dkv]] + ([tensors[g]] if self.gated else [])
        rows = sum(t.shape[0] for t in stacked)
        if rows % 8:
            stacked.append(torch.zeros(8 - rows % 8, self.hidden, dtype=tensors[q].dtype, device=tensors[q].device))
        self.w_in = torch.cat(stacked, dim=0).contiguous()
        self.q_off, self.dkv_off = 0, H * (self.dim + self.rot_dim)
        self.gate_off = self.dkv_off + self.key_width
        self.w_norm = tensors[norm]
        # U_k per head as [kv_rank, dim]: the product that carries a query into the latent's space
        self.w_uk_t = tensors[uk].view(H, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = tensors[uv].view(H, self.vdim, self.kv_rank).contiguous()
        self.w_o = tensors[o]
        self.w = {}

    def prepare(self, device, dtype):
        self.position.prepare(device, dtype)

    def subparts(self):
        return [self.position]

    # ------------------------------------------------------------------ the step
    def forward(self, ctx, h, residual, cache):
        T, H, W = h.shape[0], self.heads, self.key_width
        proj = ctx.buffer("latent_proj", (T, self.w_in.shape[0]), ctx.act_dtype)
        ops.gemm(h, self.w_in, proj)
        queries = ctx.buffer("latent_q", (T, H * W), ctx.act_dtype)
        writes = cache.writes
        ops.latent_prepare(proj, self.q_off, H, self.dim, self.rot_dim, self.dkv_off, self.kv_rank, self.w_norm, self.eps,
                           ctx.positions, self.position.freq, self.position.rotary_dim, self.position.magnitude,
                           cache.slot_mapping if writes else None, cache.k if writes else None,
                           cache.v if writes else None, queries)
        ops.head_gemm(proj, self.q_off, self.dim + self.rot_dim, self.w_uk_t, queries, 0, W)
        mixed = ctx.buffer("latent_mixed", (T, H * W), ctx.act_dtype)
        ops.attention(queries, H * W, cache.k, cache.v, cache.block_tables, ctx.attention, mixed, H, 1, W, self.window,
                      self.scale, workspace=lambda n: ctx.buffer("attention_partials", (n,), torch.float32),
                      kind=ctx.attention_kind)
        values = ctx.buffer("latent_values", (T, H * self.vdim), ctx.act_dtype)
        ops.head_gemm(mixed, 0, W, self.w_uv, values, 0, self.vdim, gate=proj if self.gated else None,
                      gate_offset=self.gate_off)
        ops.gemm(values, self.w_o, residual, accumulate=True)
