"""SiLU-gated feed-forward: down( silu(x Wg^T) * (x Wu^T) ).

gate and up are one stacked product, gate rows first (src/model/ffn.cuh:31-59,
77-84); silu(g) * u in float (src/model/activation.cuh:6-18).
"""
from __future__ import annotations

from typing import List, Mapping

import torch

from .. import ops
from .base import FEED_FORWARDS, DeferredBranch, FeedForward, Part, Runtime, StepContext, WeightSpec
from .linear import Linear


@FEED_FORWARDS.register("gated_silu")
class GatedFFN(FeedForward):
    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up = Linear([(prefix + "gate_proj.weight", intermediate_size),
                               (prefix + "up_proj.weight", intermediate_size)], hidden_size)
        self.down = Linear([(prefix + "down_proj.weight", hidden_size)], intermediate_size)

    def parts(self) -> List[Part]:
        return [self.gate_up, self.down]

    def takes_row_scale(self, n: int, ctx: StepContext) -> bool:
        return self.gate_up.gated_takes_row_scale(n)

    can_defer_last = True

    def forward(self, h: torch.Tensor, ctx: StepContext, row_scale=None, defer_last: bool = False):
        with ctx.timed("ffn_gate_up"):
            act = self.gate_up.forward_gated(h, ctx, "ffn.gate_up", row_scale=row_scale)
        if defer_last and self.down.defers(act):
            return DeferredBranch(self.down, act, ctx, "ffn.down")
        with ctx.timed("ffn_down"):
            return self.down.forward(act, ctx, "ffn.down", out_dtype=torch.float32, partials=True)


@FEED_FORWARDS.register("poly_norm")
class PolyNormFFN(FeedForward):
    """down( act(up x) ) with the PolyNorm activation act(z) = a N(z) + b N(z^2) + c N(z^3) + e: powers element by
    element, N divides a token's vector by its root mean square sqrt(mean(v^2) + eps); the four numbers are a
    checkpoint tensor.  The statistics and the polynomial are computed in float."""

    def __init__(self, up_name: str, down_name: str, act_name: str, hidden_size: int, intermediate_size: int, eps: float):
        self.hidden_size, self.intermediate_size, self.eps = hidden_size, intermediate_size, float(eps)
        self.act_name = act_name
        self.up = Linear([(up_name, intermediate_size)], hidden_size)
        self.down = Linear([(down_name, hidden_size)], intermediate_size)

    def parts(self) -> List[Part]:
        return [self.up, self.down]

    def weight_specs(self) -> List[WeightSpec]:
        return [WeightSpec(self.act_name, (4,), "poly_coefficients")]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.coef = tensors[self.act_name].to(torch.float32).contiguous()
        self.rt = rt

    def forward(self, h: torch.Tensor, ctx: StepContext):
        with ctx.timed("ffn_up"):
            # few rows: float out of the decode product (one slice: its many output rows fill the chip without a
            # split of K); many rows: the library's product in the engine's element type
            few = h.shape[0] <= ops.SKINNY_MAX_ROWS
            z = self.up.forward(h, ctx, "ffn.up", out_dtype=torch.float32 if few else None)
        act = ctx.ws.get("ffn.act", (h.shape[0], self.intermediate_size), self.rt.dtype)
        with ctx.timed("ffn_act"):
            ops.poly_norm(z, self.coef, self.eps, act)
        with ctx.timed("ffn_down"):
            return self.down.forward(act, ctx, "ffn.down", out_dtype=torch.float32, partials=True)
