"""Linear attention: a recurrent state per head instead of a cache of keys and values.

Per head, with queries and keys of ``key_dim`` elements and values of ``value_dim``:

    S_t = diag(a_t) S_(t-1) + k_t v_t^T,        o_t = S_t^T q_t

The state S (``key_dim`` x ``value_dim`` fp32 numbers a head) starts at zero and is carried from token
to token in the request's state row (``StateNeed``), so a layer of this kind holds no pages.  What
differs between designs is an option:

* ``decay``: ``"channel"``: a number per key channel that the token decides, a = sigmoid(z)^(1/tau)
  with z = W_up (W_down x) + b through a narrow inner width (``decay_down`` [r, d], ``decay_up``
  [H*key_dim, r], ``decay_bias``; r is read off the tensors), or ``"head"``: one constant per head
  (``head_decay``, a list);
* ``q_scale``: a constant on the queries;
* ``activation``: an activation on the q, k and v projections (``silu``) or none;
* ``out_norm``: the RMS norm of the result, ``"head"``: every head on its own over its ``value_dim``
  values with one weight vector [value_dim] for all heads, or ``"all"``: the heads together with a
  weight [H*value_dim];
* ``gate``: the normed result times ``silu`` or ``sigmoid`` of a projection of the input (``gate_proj``).

Then the output projection.  The decays (through their logarithm), the state, the sums over key channels
and the norm are fp32 in both dtypes; the projections take the run's dtype.
"""
from __future__ import annotations

import torch

from .base import Mixer, ParamSpec, CacheNeed, StateNeed, register
from .linear import linear, Weight
from ..csrc import hipops


@register("mixer", "linear_attention")
class LinearAttention(Mixer):
    graph_safe = True

    def __init__(self, env, hidden_size, n_heads, key_dim, value_dim, norm_eps, decay="head", head_decay=None,
                 decay_rank=16, decay_tau=1.0, q_scale=1.0, activation=None, out_norm="head", gate="silu"):
        if decay not in ("channel", "head"):
            raise ValueError(f"linear_attention: decay {decay!r} (known: channel, head)")
        if out_norm not in ("head", "all"):
            raise ValueError(f"linear_attention: out_norm {out_norm!r} (known: head, all)")
        if gate not in ("silu", "sigmoid"):
            raise ValueError(f"linear_attention: gate {gate!r} (known: silu, sigmoid)")
        if activation not in (None, "silu"):
            raise ValueError(f"linear_attention: activation {activation!r} (known: silu)")
        self.env = env
        self.d, self.H, self.D, self.V = int(hidden_size), int(n_heads), int(key_dim), int(value_dim)
        self.eps, self.q_scale, self.tau = float(norm_eps), float(q_scale), float(decay_tau)
        self.decay, self.rank, self.activation, self.out_norm, self.gate = decay, int(decay_rank), activation, out_norm, gate
        if decay == "head":
            if head_decay is None or len(head_decay) != self.H:
                raise ValueError(f"linear_attention: one constant decay for each of the {self.H} heads")
            self.head_decay_values = [float(x) for x in head_decay]
        elif not self.tau > 0:
            raise ValueError(f"linear_attention: tau = {decay_tau}")
        self.w_qkv = self.w_rest = self.w_up = self.wo = self.w_norm = self.b_decay = self.head_decay = None

    # ------------------------------------------------------------------ tensors
    def params(self):
        d, HD, HV = self.d, self.H * self.D, self.H * self.V
        p = {"q_proj": ParamSpec((HD, d)), "k_proj": ParamSpec((HD, d)), "v_proj": ParamSpec((HV, d)),
             "gate_proj": ParamSpec((HV, d)), "o_proj": ParamSpec((d, HV)),
             "norm": ParamSpec((self.V if self.out_norm == "head" else HV,), kind="vector", init="ones")}
        if self.decay == "channel":
            p.update({"decay_down": ParamSpec((self.rank, d), free=(0,)), "decay_up": ParamSpec((HD, self.rank), free=(1,)),
                      "decay_bias": ParamSpec((HD,), kind="vector", init="normal")})
        return p

    @staticmethod
    def _stack(mats):
        """Matrices of one input width one under the other, in one dtype, padded to whole bands of 16 rows
        (so that the weight can be kept in operand order)."""
        dts = {m.dtype for m in mats}
        dt = torch.float32 if len(dts) > 1 else dts.pop()
        w = torch.cat([m.to(dt) for m in mats], dim=0)
        pad = -w.shape[0] % 16
        if pad:
            w = torch.cat([w, torch.zeros((pad, w.shape[1]), dtype=dt, device=w.device)], dim=0)
        return w

    def load(self, t):
        qkv = [t["q_proj"], t["k_proj"], t["v_proj"]]
        rest = [t["gate_proj"]]
        if self.decay == "channel":
            self.rank = int(t["decay_down"].shape[0])
            if t["decay_up"].shape[1] != self.rank:
                raise ValueError(f"linear_attention: the decay's two matrices meet in {self.rank} and {t['decay_up'].shape[1]} elements")
            # the decay's narrow rows come first: the second product reads them as a column range of the
            # first one's result, which then starts where a row starts
            rest.insert(0, t["decay_down"])
            self.w_up = Weight(t["decay_up"])
            self.b_decay = t["decay_bias"].float().contiguous()
        else:
            self.rank = 0
            self.head_decay = torch.tensor(self.head_decay_values, dtype=torch.float64).to(torch.float32).to(self.env.device)
        if self.activation is None:
            # one product for everything that reads the mixer's input: [decay | gate | q | k | v]
            self.w_qkv, self.w_rest = Weight(self._stack(rest + qkv)), None
        else:
            # the activation is the epilogue of the q/k/v product; gate and decay rows have none
            self.w_qkv, self.w_rest = Weight(self._stack(qkv)), Weight(self._stack(rest))
        self.wo = Weight(t["o_proj"])
        self.w_norm = t["norm"].float().contiguous()

    def slow_paths(self, page_size):
        notes = []
        if self.env.dtype == torch.bfloat16:
            for name, w in (("q/k/v projection", self.w_qkv), ("gate projection", self.w_rest), ("decay projection", self.w_up),
                            ("output projection", self.wo)):
                if w is not None:
                    notes += w.slow_reason(name)
        return notes

    def cache_need(self):
        return CacheNeed(state=StateNeed((self.H, self.D, self.V), torch.float32))

    # ------------------------------------------------------------------ the step
    def forward(self, x, ctx, cache):
        T, ws = x.shape[0], ctx.ws
        H, D, V = self.H, self.D, self.V
        HD, HV = H * D, H * V
        r = self.rank
        proj = ws.take((T, self.w_qkv.shape[0]), x.dtype)
        linear(x, self.w_qkv, proj, ws=ws, act=self.activation)
        if self.w_rest is None:
            rest, qkv = proj, proj[:, r + HV:]
        else:
            rest, qkv = ws.take((T, self.w_rest.shape[0]), x.dtype), proj
            linear(x, self.w_rest, rest, ws=ws)
        decay = None
        if self.decay == "channel":
            decay = ws.take((T, HD), torch.float32)
            linear(rest[:, :r], self.w_up, decay, ws=ws)
            hipops.channel_decay(decay, self.b_decay, self.tau)
        o = ws.take((T, HV), torch.float32)
        hipops.linear_attn_scan(qkv[:, :HD], qkv[:, HD:2 * HD], qkv[:, 2 * HD:2 * HD + HV], o, cache.state,
                                ctx.cu_seqlens, ctx.seq_slots, ctx.n_seqs, H, D, V, decay=decay,
                                head_decay=self.head_decay, q_scale=self.q_scale, longest=ctx.max_count)
        y = ws.take((T, HV), x.dtype)
        hipops.gated_group_norm(o, self.w_norm, y, V if self.out_norm == "head" else HV, self.eps,
                                gate=rest[:, r:r + HV], act=self.gate)
        out = ws.take((T, self.d), torch.float32)
        linear(y, self.wo, out, ws=ws)
        return out
