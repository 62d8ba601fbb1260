"""A state-space mixer in the "state-space duality" form: a scalar decay per head and token.

With inner = heads * vdim, N = ``state`` channels and G ``groups`` (head h reads group h // (heads / G)), the input
projection's row is [z: inner | x: inner | B: G*N | C: G*N | dt: heads].  x, B and C pass a short causal convolution
per channel (weights [channels, taps] and a bias, the last column the token's own) and silu.  Then, per head,

    dt = softplus(dt + dt_bias)                       the step size (no clamp)
    S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T  S: N x vdim
    y_t = S_t^T C_t + D x_t

y (heads concatenated) times silu(z), then an RMS norm in ``norm_groups`` equal parts, times ``norm``, then the output
projection: the gate comes before the norm.  The state S and the convolution's last taps - 1 inputs are kept between
steps in two state tensors (``state`` and ``conv``).  Step sizes, decays, the recurrence and the norm are fp32 in both
dtypes; projections and the convolution's results take the run's dtype.
"""
from __future__ import annotations

import torch

from .base import Mixer, ParamSpec, CacheNeed, StateNeed, register
from .linear import linear, Weight
from ..csrc import hipops


@register("mixer", "state_space")
class StateSpace(Mixer):
    graph_safe = True

    def __init__(self, env, hidden_size, n_heads, value_dim, state_dim, n_groups, conv_taps, norm_groups, norm_eps):
        self.env = env
        self.d, self.H, self.P, self.N, self.G = int(hidden_size), int(n_heads), int(value_dim), int(state_dim), int(n_groups)
        self.taps, self.parts, self.eps = int(conv_taps), int(norm_groups), float(norm_eps)
        self.inner = self.H * self.P
        if self.H % self.G:
            raise ValueError(f"state_space: {self.H} heads over {self.G} groups")
        if self.inner % self.parts:
            raise ValueError(f"state_space: {self.inner} inner channels in {self.parts} norm groups")
        if self.N > 256:
            raise ValueError(f"state_space: {self.N} state channels (at most 256)")
        if self.taps < 1:
            raise ValueError(f"state_space: a convolution of {self.taps} taps")
        self.n_conv = self.inner + 2 * self.G * self.N
        self.n_in = 2 * self.inner + 2 * self.G * self.N + self.H
        self.w_in = self.w_conv = self.b_conv = self.dt_bias = self.a_log = self.skip = self.w_norm = self.wo = None

    def params(self):
        return {"in_proj": ParamSpec((self.n_in, self.d)), "conv": ParamSpec((self.n_conv, self.taps), kind="vector", init="normal"),
                "conv_bias": ParamSpec((self.n_conv,), kind="vector", init="normal"),
                "dt_bias": ParamSpec((self.H,), kind="vector", init="normal"), "a_log": ParamSpec((self.H,), kind="vector", init="normal"),
                "skip": ParamSpec((self.H,), kind="vector", init="ones"),
                "norm": ParamSpec((self.inner,), kind="vector", init="ones"), "o_proj": ParamSpec((self.d, self.inner))}

    def load(self, t):
        w = t["in_proj"]
        pad = -w.shape[0] % 16               # whole bands of 16 rows: the weight can be kept in operand order
        if pad:
            w = torch.cat([w, torch.zeros((pad, w.shape[1]), dtype=w.dtype, device=w.device)], dim=0)
        self.rows_in = w.shape[0]
        self.w_in = Weight(w)
        # tap by tap, [taps, channels]: the kernel's loads of one tap are consecutive
        self.w_conv, self.b_conv = t["conv"].float().t().contiguous(), t["conv_bias"].float().contiguous()
        self.dt_bias, self.a_log = t["dt_bias"].float().contiguous(), t["a_log"].float().contiguous()
        self.skip, self.w_norm = t["skip"].float().contiguous(), t["norm"].float().contiguous()
        self.wo = Weight(t["o_proj"])

    def slow_paths(self, page_size):
        notes = []
        if self.env.dtype == torch.bfloat16 and self.w_in is not None:
            notes += self.w_in.slow_reason("input projection") + self.wo.slow_reason("output projection")
        return notes

    def cache_needs(self):
        needs = {"state": CacheNeed(state=StateNeed((self.H, self.N, self.P), torch.float32))}
        if self.taps > 1:
            needs["conv"] = CacheNeed(state=StateNeed((self.taps - 1, self.n_conv), torch.float32))
        return needs

    def forward(self, x, ctx, cache):
        T, ws = x.shape[0], ctx.ws
        H, P, N, G, inner = self.H, self.P, self.N, self.G, self.inner
        proj = ws.take((T, self.rows_in), x.dtype)
        linear(x, self.w_in, proj, ws=ws)
        xbc = ws.take((T, self.n_conv), x.dtype)
        hipops.causal_conv(proj[:, inner:inner + self.n_conv], self.w_conv, xbc, cache["conv"].state if self.taps > 1 else None,
                           ctx.seq_of_token, ctx.cu_seqlens, ctx.seq_slots, bias=self.b_conv, act="silu")
        dt = ws.take((T, H), torch.float32)
        decay = ws.take((T, H * N), torch.float32)
        hipops.step_decay(proj[:, inner + self.n_conv:inner + self.n_conv + H], self.dt_bias, self.a_log, dt, decay, H, N)
        y = ws.take((T, inner), torch.float32)
        # C is the recurrence's query, B its key (both shared by the heads of a group), x its value, dt the factor on it
        hipops.linear_attn_scan(xbc[:, inner + G * N:], xbc[:, inner:inner + G * N], xbc[:, :inner], y, cache["state"].state,
                                ctx.cu_seqlens, ctx.seq_slots, ctx.n_seqs, H, N, P, decay=decay, qk_heads=G, v_scale=dt,
                                longest=ctx.max_count)
        g = ws.take((T, inner), x.dtype)
        hipops.gated_group_norm(y, self.w_norm, g, inner // self.parts, self.eps, gate=proj[:, :inner], act="silu", gate_first=True,
                                skip=xbc[:, :inner], skip_weight=self.skip, skip_group=P)
        out = ws.take((T, self.d), torch.float32)
        linear(g, self.wo, out, ws=ws)
        return out
