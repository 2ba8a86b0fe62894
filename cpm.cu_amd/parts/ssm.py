"""State-space mixer of the Mamba-2 kind (state-space duality): a gated linear recurrence with a matrix state.

With inner = heads * head_dim, N = state_size, G = groups, one input projection gives
[z: inner | x: inner | B: G*N | C: G*N | dt: heads] per token.  x, B and C pass a causal convolution per
channel (``conv_taps`` taps, the last one the current token's, zeros before the sequence's start, with bias)
and SiLU.  Per head h, with group g = h // (heads / G):

    d_t = softplus(dt_t + dt_bias[h])                      (no clamp)
    S_t = exp(-exp(A_log[h]) * d_t) * S_(t-1) + d_t * B_t x_t^T          S: [N, head_dim], zero at the start
    y_t = S_t^T C_t + D[h] * x_t

y (heads side by side) is multiplied by silu(z), then RMS-normed in ``norm_groups`` equal parts (each by its
own root mean square) times a weight, then projected out.  The gate comes before the norm.

Everything after the convolution runs in float; the recurrent state and the convolution's last
``conv_taps - 1`` inputs live as float fixed-size state in the sequence's cache slot, so a step of any number
of tokens continues where the last one ended.
"""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from .. import ops
from ..cache.paged import CacheNeeds, CacheView, StateSpec
from .base import MIXERS, Mixer, Part, Runtime, StepContext, WeightSpec
from .linear import Linear


@MIXERS.register("mamba2")
class Mamba2Mixer(Mixer):
    def __init__(self, names: Mapping[str, str], hidden_size: int, heads: int, head_dim: int, state_size: int,
                 groups: int, conv_taps: int, norm_groups: int, eps: float):
        """``names``: checkpoint tensors for 'in', 'conv', 'conv_bias', 'dt_bias', 'A_log', 'D', 'norm', 'out'."""
        if heads % groups:
            raise ValueError(f"mamba2: {heads} heads are not a multiple of {groups} groups")
        inner = heads * head_dim
        if inner % norm_groups:
            raise ValueError(f"mamba2: {inner} inner features do not split into {norm_groups} norm groups")
        if state_size > 256:
            raise ValueError(f"mamba2: a state of {state_size} values a feature is not supported (at most 256)")
        if conv_taps < 1:
            raise ValueError(f"mamba2: {conv_taps} convolution taps")
        self.names = dict(names)
        self.hidden_size, self.heads, self.head_dim, self.state_size = hidden_size, heads, head_dim, state_size
        self.groups, self.taps, self.norm_groups, self.eps = groups, conv_taps, norm_groups, float(eps)
        self.inner = inner
        self.channels = inner + 2 * groups * state_size
        self.in_proj = Linear([(self.names["in"], 2 * inner + 2 * groups * state_size + heads)], hidden_size)
        self.out_proj = Linear([(self.names["out"], hidden_size)], inner)

    def parts(self) -> List[Part]:
        return [self.in_proj, self.out_proj]

    def weight_specs(self) -> List[WeightSpec]:
        n = self.names
        return [WeightSpec(n["conv"], (self.channels, self.taps), "conv_taps"),
                WeightSpec(n["conv_bias"], (self.channels,), "small"),
                WeightSpec(n["dt_bias"], (self.heads,), "small"),
                WeightSpec(n["A_log"], (self.heads,), "log_decay"),
                WeightSpec(n["D"], (self.heads,), "norm"),
                WeightSpec(n["norm"], (self.inner,), "norm")]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        f = lambda k: tensors[self.names[k]].to(torch.float32).contiguous()
        self.conv_w, self.conv_b = f("conv"), f("conv_bias")
        self.dt_bias, self.A_log, self.D, self.norm_w = f("dt_bias"), f("A_log"), f("D"), f("norm")
        self.rt = rt

    def cache_needs(self) -> CacheNeeds:
        state = [("ssm", StateSpec((self.heads, self.head_dim, self.state_size), torch.float32))]
        if self.taps > 1:
            state.append(("conv", StateSpec((self.taps - 1, self.channels), torch.float32)))
        return CacheNeeds(state=tuple(state))

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        n, inner = h.shape[0], self.inner
        with ctx.timed("ssm_in"):
            u = self.in_proj.forward(h, ctx, "ssm.in")
        xbc = ctx.ws.get("ssm.xbc", (n, self.channels), torch.float32)
        y = ctx.ws.get("ssm.y", (n, inner), torch.float32)
        with ctx.timed("ssm_conv"):
            ops.conv_silu(u[:, inner:inner + self.channels], self.conv_w, self.conv_b, cache.state.get("conv"), xbc,
                          ctx.cu_q, ctx.seq_slot, max(ctx.q_lens), update_state=writes_cache)
        with ctx.timed("ssm_scan"):
            ops.ssm_scan(xbc, u[:, inner + self.channels:], self.dt_bias, self.A_log, self.D, cache.state["ssm"], y,
                         ctx.cu_q, ctx.seq_slot, self.heads, self.head_dim, self.state_size, self.groups,
                         write_state=writes_cache)
        gated = ctx.ws.get("ssm.gated", (n, inner), self.rt.dtype)
        with ctx.timed("ssm_norm"):
            ops.rms_norm_groups(y, self.norm_w, self.eps, gated, groups=self.norm_groups, gate=u[:, :inner])
        with ctx.timed("ssm_out"):
            return self.out_proj.forward(gated, ctx, "ssm.out", out_dtype=torch.float32, partials=True)
