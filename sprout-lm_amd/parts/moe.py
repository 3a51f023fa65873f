"""A feed-forward of routed experts, with an optional shared expert that every token takes."""
from __future__ import annotations

import torch

from .. import ops
from ..config.base import ConfigError
from ..weights.loader import TensorSpec
from .base import FeedForward, register_part
from .mlp import GatedMLP


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    """y = sum over a token's `top` experts of weight_e * down_e(act(gate_e x) * up_e x)  (+ shared(x)).

    Router logits z = W_r x + b are float32; the `top` largest are chosen (the lowest index wins a tie) and their
    weights are the softmax over the chosen logits alone.  Nothing is decided on the host: a kernel makes the choice,
    sorts the (token, choice) pairs by expert and cuts every expert's rows into tiles, the two grouped products walk those
    tiles (the first gathers its rows from the tokens and applies the activation, the second writes float32 rows),
    and the weighted sum is taken per token in the order of its choices, so a token's result does not depend on what
    else is in the step.

    hidden, inner, experts, top: sizes.  shared_inner: inner size of the shared expert (None: there is none).
    router_bias: whether the router has a bias.  `tensors`: local name patterns of an expert's gate, up and down
    matrices (`{e}` = the expert's number), of the router's weight and bias, and the prefix of the shared expert.
    """

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, inner: int, experts: int, top: int, shared_inner: int | None = None,
                 router_bias: bool = True, activation: str = "silu",
                 tensors: tuple = ("e{e}.gate", "e{e}.up", "e{e}.down", "router", "router.b", "shared.")):
        if min(hidden, inner, experts, top) <= 0 or top > experts:
            raise ConfigError(f"A routed feed-forward needs 0 < top <= experts and positive sizes, got top={top} "
                              f"experts={experts} inner={inner}.")
        if activation not in ops.GATE_ACTIVATIONS:
            raise ConfigError(f"Experts with activation {activation!r} have no kernel; there are kernels for "
                              f"{sorted(ops.GATE_ACTIVATIONS)}.")
        self.hidden, self.inner, self.experts, self.top = hidden, inner, experts, top
        self.router_bias, self.activation, self.names = router_bias, activation, tuple(tensors)
        prefix = self.names[5]
        self.shared = None if not shared_inner else GatedMLP(hidden, shared_inner, activation,
                                                             tensors=(prefix + "gate", prefix + "up", prefix + "down"))

    def subparts(self):
        return [self.shared] if self.shared is not None else []

    def flops(self, tokens: int, pairs: int = 0) -> float:
        total = 2.0 * tokens * self.hidden * (self.experts + 3 * self.inner * self.top)
        return total + (self.shared.flops(tokens) if self.shared is not None else 0.0)

    def tensors(self):
        gate, up, down, router, bias, _ = self.names
        out = {}
        for e in range(self.experts):
            out[gate.format(e=e)] = TensorSpec((self.inner, self.hidden))
            out[up.format(e=e)] = TensorSpec((self.inner, self.hidden))
            out[down.format(e=e)] = TensorSpec((self.hidden, self.inner))
        out[router] = TensorSpec((self.experts, self.hidden))
        if self.router_bias:
            out[bias] = TensorSpec((self.experts,), "vector")
        if self.shared is not None:
            out.update(self.shared.tensors())
        return out

    def bind(self, tensors):
        gate, up, down, router, bias, _ = self.names
        E = self.experts
        # [experts, 2 inner, hidden]: an expert's gate rows, then its up rows; [experts, hidden, inner]
        self.w_gate_up = torch.stack([torch.cat([tensors.pop(gate.format(e=e)), tensors.pop(up.format(e=e))], dim=0)
                                      for e in range(E)]).contiguous()
        self.w_down = torch.stack([tensors.pop(down.format(e=e)) for e in range(E)]).contiguous()
        self.w_router = tensors[router]
        self.b_router = tensors[bias] if self.router_bias else None
        if self.shared is not None:
            self.shared.bind({name: tensors[name] for name in self.shared.tensors()})
        self.w = {}

    def forward(self, ctx, h, residual):
        T, E, top = h.shape[0], self.experts, self.top
        pairs = T * top
        logits = ctx.buffer("router_logits", (T, E), torch.float32)
        ops.gemm(h, self.w_router, logits, bias=self.b_router)
        ids = ctx.buffer("expert_ids", (T, top), torch.int32)
        weights = ctx.buffer("expert_weights", (T, top), torch.float32)
        row_of_pair = ctx.buffer("expert_row_of_pair", (pairs,), torch.int32)
        pair_of_row = ctx.buffer("expert_pair_of_row", (pairs,), torch.int32)
        tile_rows = ops.group_tile_rows(ctx.act_dtype, pairs, E, self.hidden % 8 == 0 and self.inner % 8 == 0)
        tiles = ctx.buffer("expert_tiles", (3 * ops.route_max_tiles(pairs, E, tile_rows),), torch.int32)
        n_tiles = ctx.buffer("expert_tile_count", (1,), torch.int32)
        ops.route(logits, ids, weights, row_of_pair, pair_of_row, tiles, n_tiles, tile_rows)
        act = ctx.buffer("expert_act", (pairs, self.inner), ctx.act_dtype)
        ops.expert_gate_up(h, self.w_gate_up, tiles, n_tiles, pair_of_row, top, act, activation=self.activation,
                           tile_rows=tile_rows)
        out = ctx.buffer("expert_out", (pairs, self.hidden), torch.float32)
        ops.expert_down(act, self.w_down, tiles, n_tiles, out, tile_rows=tile_rows)
        ops.route_combine(out, row_of_pair, weights, residual)
        if self.shared is not None:
            self.shared.forward(ctx, h, residual)
