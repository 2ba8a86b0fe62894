"""Matrix-memory recurrent mixer of the mLSTM kind (xLSTM's matrix LSTM): a gated linear recurrence whose state
is a matrix a head, with exponential gates kept in range by a running maximum.

One input projection gives [q: heads*dim | k: heads*dim | v: heads*vdim | g: heads*vdim | i: heads | f: heads] per
token.  Per head, with q scaled by dim^-1/2:

    a_t = cap tanh((i_t + bi) / cap)                   log input gate
    b_t = logsigmoid(cap tanh((f_t + bf) / cap))       log forget gate
    m_t = max(b_t + m_(t-1), a_t)                      m starts at 0
    S_t = exp(b_t + m_(t-1) - m_t) S_(t-1) + exp(a_t - m_t) k_t v_t^T        S, n start at 0
    n_t = exp(b_t + m_(t-1) - m_t) n_(t-1) + exp(a_t - m_t) k_t
    y_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)

Each head's y is divided by its root mean square; the heads side by side are multiplied by a weight, then by
sigmoid(g) (the gate comes after the norm), then projected out.

Everything after the projection runs in float; S, n and m live as float fixed-size state in the sequence's cache
slot, so a step of any number of tokens continues where the last one ended.
"""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .. import ops
from ..cache.paged import CacheNeeds, CacheView, StateSpec
from .base import MIXERS, Mixer, Part, Runtime, StepContext, WeightSpec
from .linear import Linear


@MIXERS.register("mlstm")
class MLSTMMixer(Mixer):
    def __init__(self, names: Mapping[str, str], hidden_size: int, heads: int, key_dim: int, value_dim: int,
                 gate_cap: float, eps: float):
        """``names``: checkpoint tensors for 'q', 'k', 'v', 'gate', 'input_gate', 'input_gate_bias', 'forget_gate',
        'forget_gate_bias', 'norm', 'out'."""
        if key_dim > 1024:
            raise ValueError(f"mlstm: a key size of {key_dim} is not supported (at most 1024)")
        if gate_cap <= 0:
            raise ValueError(f"mlstm: gate cap {gate_cap}")
        self.names = dict(names)
        self.hidden_size, self.heads, self.dk, self.dv = hidden_size, heads, key_dim, value_dim
        self.cap, self.eps = float(gate_cap), float(eps)
        n = self.names
        self.in_proj = Linear([(n["q"], heads * key_dim), (n["k"], heads * key_dim), (n["v"], heads * value_dim),
                               (n["gate"], heads * value_dim), (n["input_gate"], heads), (n["forget_gate"], heads)],
                              hidden_size)
        self.out_proj = Linear([(n["out"], hidden_size)], heads * value_dim)
        hk, hv = heads * key_dim, heads * value_dim
        self.q_off, self.k_off, self.v_off, self.g_off = 0, hk, 2 * hk, 2 * hk + hv
        self.i_off, self.f_off = 2 * hk + 2 * hv, 2 * hk + 2 * hv + heads

    def parts(self) -> List[Part]:
        return [self.in_proj, self.out_proj]

    def weight_specs(self) -> List[WeightSpec]:
        n = self.names
        return [WeightSpec(n["input_gate_bias"], (self.heads,), "small"),
                WeightSpec(n["forget_gate_bias"], (self.heads,), "small"),
                WeightSpec(n["norm"], (self.heads * self.dv,), "norm")]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        f = lambda k: tensors[self.names[k]].to(torch.float32).contiguous()
        self.i_bias, self.f_bias, self.norm_w = f("input_gate_bias"), f("forget_gate_bias"), f("norm")
        self.rt = rt

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(state=(("memory", StateSpec((self.heads, self.dv, self.dk), torch.float32)),
                                 ("normaliser", StateSpec((self.heads, self.dk), torch.float32)),
                                 ("maximum", StateSpec((self.heads,), torch.float32))))

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        n, hv = h.shape[0], self.heads * self.dv
        with ctx.timed("mlstm_in"):
            u = self.in_proj.forward(h, ctx, "mlstm.in")
        y = ctx.ws.get("mlstm.y", (n, hv), torch.float32)
        den = ctx.ws.get("mlstm.den", (n, self.heads), torch.float32)
        with ctx.timed("mlstm_scan"):
            ops.mlstm_scan(u, self.q_off, self.k_off, self.v_off, self.i_off, self.f_off, self.i_bias, self.f_bias,
                           self.cap, self.dk ** -0.5, cache.state["memory"], cache.state["normaliser"],
                           cache.state["maximum"], y, den, ctx.cu_q, ctx.seq_slot, self.heads, self.dk, self.dv,
                           write_state=writes_cache)
        gated = ctx.ws.get("mlstm.gated", (n, hv), self.rt.dtype)
        with ctx.timed("mlstm_norm"):
            ops.rms_norm_groups(y, self.norm_w, self.eps, gated, groups=self.heads,
                                gate=u[:, self.g_off:self.g_off + hv], gate_after=True, divisor=den)
        with ctx.timed("mlstm_out"):
            return self.out_proj.forward(gated, ctx, "mlstm.out", out_dtype=torch.float32, partials=True)
