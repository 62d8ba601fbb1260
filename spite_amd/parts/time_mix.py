"""Time mixing with a decayed state per head (the RWKV family's form of linear attention).

With x' the row of the token before (zeros before a request's first token), each of the five readers
s in (r, k, v, g, w) reads its own blend  x + (x' - x) * mu_s.  Per head of ``dim`` channels:

    r, k, v = W_r, W_k, W_v of their blends;      gate = silu(W_g blend_g)
    w = exp(-exp(W_w2 tanh(W_w1 blend_w) + w0))   the decay, a number per key channel and token
    o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t     u: a bonus for the token's own outer product
    S_t = diag(w_t) S_(t-1) + k_t v_t^T

Every head's o is divided by its root mean square, the heads are concatenated, times ``norm``, times the gate, then
the output projection.  The state S (``dim`` x ``dim`` fp32 numbers a head) and the request's last input row are
kept between steps in two state tensors (``state`` and ``shift``).  Blends, decays, the recurrence and the norm are
fp32 in both dtypes; the projections take the run's dtype.
"""
from __future__ import annotations

import torch

from .base import Mixer, ParamSpec, CacheNeed, StateNeed, register
from .linear import linear, Weight
from ..csrc import hipops

READERS = ("r", "k", "v", "g", "w")


@register("mixer", "time_mix")
class TimeMix(Mixer):
    graph_safe = True

    def __init__(self, env, hidden_size, n_heads, head_dim, norm_eps, decay_rank=16):
        self.env = env
        self.d, self.H, self.D, self.eps, self.rank = int(hidden_size), int(n_heads), int(head_dim), float(norm_eps), int(decay_rank)
        if self.D > 256:
            raise ValueError(f"time_mix: heads of {self.D} channels (at most 256)")
        self.mu = self.w = self.w_down = self.w_up = self.w0 = self.u = self.w_norm = self.wo = None

    def params(self):
        d, n = self.d, self.H * self.D
        p = {f"mu_{s}": ParamSpec((d,), kind="vector", init="normal") for s in READERS}
        p.update({f"{s}_proj": ParamSpec((n, d)) for s in ("r", "k", "v", "g")})
        p.update({"decay_down": ParamSpec((self.rank, d), free=(0,)), "decay_up": ParamSpec((n, self.rank), free=(1,)),
                  "decay_bias": ParamSpec((n,), kind="vector", init="normal"),
                  "bonus": ParamSpec((self.H, self.D), kind="vector", init="normal"),
                  "norm": ParamSpec((n,), kind="vector", init="ones"), "o_proj": ParamSpec((d, n))})
        return p

    def load(self, t):
        self.rank = int(t["decay_down"].shape[0])
        if t["decay_up"].shape[1] != self.rank:
            raise ValueError(f"time_mix: the decay's two matrices meet in {self.rank} and {t['decay_up'].shape[1]} elements")
        self.mu = torch.stack([t[f"mu_{s}"].float() for s in READERS]).contiguous()
        self.w = {s: Weight(t[f"{s}_proj"]) for s in ("r", "k", "v", "g")}
        self.w_down, self.w_up = Weight(t["decay_down"]), Weight(t["decay_up"])
        self.w0 = t["decay_bias"].float().contiguous()
        self.u = t["bonus"].float().contiguous()
        self.w_norm = t["norm"].float().contiguous()
        self.wo = Weight(t["o_proj"])

    def slow_paths(self, page_size):
        notes = []
        if self.env.dtype == torch.bfloat16 and self.w is not None:
            for name, w in [(f"{s} projection", w) for s, w in self.w.items()] + [("decay projections", self.w_down), ("output projection", self.wo)]:
                notes += w.slow_reason(name)
        return notes

    def cache_needs(self):
        return {"state": CacheNeed(state=StateNeed((self.H, self.D, self.D), torch.float32)),
                "shift": CacheNeed(state=StateNeed((self.d,), torch.float32))}

    def forward(self, x, ctx, cache):
        T, ws = x.shape[0], ctx.ws
        H, D, n = self.H, self.D, self.H * self.D
        blends = ws.take((len(READERS), T, self.d), x.dtype)
        hipops.shift_mix(x, self.mu, cache["shift"].state, blends, ctx.seq_of_token, ctx.cu_seqlens, ctx.seq_slots)
        rkvg = ws.take((4, T, n), x.dtype)
        for i, s in enumerate(("r", "k", "v", "g")):
            linear(blends[i], self.w[s], rkvg[i], ws=ws)
        low = ws.take((T, self.rank), x.dtype)
        linear(blends[4], self.w_down, low, ws=ws, act="tanh")
        decay = ws.take((T, n), torch.float32)
        linear(low, self.w_up, decay, ws=ws)
        hipops.channel_decay(decay, self.w0, form="exp_exp")
        o = ws.take((T, n), torch.float32)
        hipops.linear_attn_scan(rkvg[0], rkvg[1], rkvg[2], o, cache["state"].state, ctx.cu_seqlens, ctx.seq_slots, ctx.n_seqs,
                                H, D, D, decay=decay, bonus=self.u, longest=ctx.max_count)
        y = ws.take((T, n), x.dtype)
        hipops.gated_group_norm(o, self.w_norm, y, D, self.eps, gate=rkvg[3], act="silu")
        out = ws.take((T, self.d), torch.float32)
        linear(y, self.wo, out, ws=ws)
        return out
