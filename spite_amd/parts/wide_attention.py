"""Attention whose keys and values differ in shape, with the options that stand around it.

``wide_attention`` is grouped-query attention over the paged cache, H query heads on G kv heads,
keys and queries ``key_dim`` wide, values ``value_dim`` wide, with, each as an option:

* ``bias``: q, k and v projections with biases (``q_bias``, ``k_bias``, ``v_bias``);
* ``projection_norm``: an RMS norm over the whole q projection and over the whole k projection
  (all heads at once, weights ``q_norm`` [H*key_dim] and ``k_norm`` [G*key_dim]) before the rotation;
* the position encoding of q and k (a ``position`` part; its first ``rotary_dim`` elements turn);
* ``value_position``: the values turn by their own position before they are cached, over all of
  ``value_dim``, and every head's result is turned back by the query's position: value j reaches
  query i turned by j - i;
* ``maps`` = 2, differential attention: every head has two queries and two keys (rows laid out
  head by head as [map 1 | map 2]); each map is a softmax attention of its own over the same
  values, and the head's result is ``a1 - lambda * a2`` divided by its root mean square over the
  head's values, times ``1 - diff``; lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff is one number
  of the layer, formed from four vectors of the checkpoint when it is loaded;
* ``head_gate``: head h's result times sigmoid(W_g x)_h (``gate_proj`` [H, d]), before the output
  projection;
* ``sinks``: every head's softmax has one more term in its denominator, exp(s_h) with a learned number
  s_h per head (``sink`` [H]): it is no key, is not scaled, brings no value and counts once, so a head
  may give less than all of its weight to the keys it sees; ``sinks="zero"``: the term is exp(0) = 1 for
  every head and no tensor holds it;
* ``conv_taps`` >= 1: a short causal convolution over time on every channel of the q and of the k projection
  (``q_conv`` [H*key_dim, taps], ``k_conv`` [G*key_dim, taps], the last column the token's own), right after the
  projection; the last taps - 1 projected rows of a request are its state between steps;
* ``head_norm``: an RMS norm of every q and k head on its own, with one weight vector for all heads
  (``q_norm``, ``k_norm`` [key_dim]);
* ``q_temperature`` = (coef, every): the normed queries at position p times 1 + coef ln(floor((p+1)/every) + 1);
* ``values="keys"``: there is no value projection; the values are the keys as they leave the convolution,
  before their norm (``value_dim`` = ``key_dim``);
* ``score_position``: a position part that works on the scores (per-head slopes on the distance).

Inside, two maps are 2H query heads over 2G key heads over G value heads: the projections' rows
are reordered map by map when they are loaded, so that query head m*H + h reads key head
m*G + g and value head g.  Scores, softmax, the sums over the values, norms, angles and the gate's
sigmoid are fp32 in both dtypes.
"""
from __future__ import annotations

import math

import torch

from .base import Mixer, ParamSpec, CacheNeed, KVNeed, register, build as build_part
from .attention import TAIL
from .linear import linear, Weight
from ..csrc import hipops


@register("mixer", "wide_attention")
class WideAttention(Mixer):
    graph_safe = True
    step_arrays = (TAIL,)

    def __init__(self, env, hidden_size, n_heads, n_kv_heads, key_dim, value_dim, scale, position=None,
                 value_position=None, visibility="full", span=0, bias=False, projection_norm=False, norm_eps=1e-5,
                 maps=1, diff=0.0, head_gate=False, sinks=False, conv_taps=0, head_norm=False, q_temperature=None,
                 values="projection", score_position=None):
        if n_heads % n_kv_heads:
            raise ValueError(f"wide_attention: {n_heads} heads over {n_kv_heads} kv heads")
        if visibility not in hipops.VIS:
            raise ValueError(f"wide_attention: visibility {visibility!r} (known: {sorted(hipops.VIS)})")
        if visibility != "full" and span < 1:
            raise ValueError(f"wide_attention: {visibility} of size {span}")
        if maps not in (1, 2):
            raise ValueError(f"wide_attention: {maps} score maps a head")
        if maps == 2 and (value_position is not None or head_gate or sinks):
            raise ValueError("wide_attention: two score maps go with neither turned values nor a head gate nor sinks")
        if values not in ("projection", "keys"):
            raise ValueError(f"wide_attention: values {values!r} (known: projection, keys)")
        if values == "keys" and (int(value_dim) != int(key_dim) or maps != 1 or value_position is not None or bias):
            raise ValueError("wide_attention: values taken from the keys have the keys' width, one map, no rotation, no bias")
        if head_norm and projection_norm:
            raise ValueError("wide_attention: a norm per head or one over the whole projection, not both")
        if (conv_taps or 0) >= 1 and (maps != 1 or bias or values != "keys"):
            raise ValueError("wide_attention: the convolution goes with one map, no biases and values taken from the keys")
        if sinks not in (False, True, None, "zero"):
            raise ValueError(f"wide_attention: sinks {sinks!r} (known: True, 'zero')")
        self.env = env
        self.d, self.H, self.G = int(hidden_size), int(n_heads), int(n_kv_heads)
        self.D, self.Vd, self.maps = int(key_dim), int(value_dim), int(maps)
        self.scale, self.diff, self.eps = float(scale), float(diff), float(norm_eps)
        self.visibility, self.span = visibility, int(span or 0)
        self.bias, self.projection_norm, self.head_gate = bool(bias), bool(projection_norm), bool(head_gate)
        self.sinks = bool(sinks)
        self.zero_sinks = sinks == "zero"
        self.w_sink = None
        self.taps = max(int(conv_taps or 0), 0)             # 1: a weight per channel on the token's own row, no state
        self.head_norm, self.values_from_keys = bool(head_norm), values == "keys"
        self.q_temperature = None if not q_temperature else (float(q_temperature[0]), int(q_temperature[1]))
        if self.q_temperature is not None and self.q_temperature[1] < 1:
            raise ValueError(f"wide_attention: query temperature every {self.q_temperature[1]} positions")
        self.score_position = build_part("position", score_position, env) if score_position is not None else None
        self.slopes = self.w_conv = None
        self.position = build_part("position", position, env) if position is not None else None
        self.value_position = build_part("position", value_position, env) if value_position is not None else None
        for pe in (self.position, self.value_position):
            if pe is not None and (not pe.fused or pe.kernel_args().get("adjacent")):
                raise ValueError("wide_attention: the position encoding must be a rotation in halves")
        self.HQ, self.GK = self.H * self.maps, self.G * self.maps
        # the MFMA kernels take keys and values of one width, 64 or 128: narrower keys (and queries) are stored
        # that wide in a bfloat16 run, zeros behind their own elements
        self.Dk = self.D
        if env.dtype == torch.bfloat16 and self.Vd in (64, 128) and self.D < self.Vd and self.HQ // self.GK <= 16:
            self.Dk = self.Vd
        self.n_qk = (self.HQ + self.GK) * self.D
        self.n_qkv = self.n_qk + (0 if self.values_from_keys else self.G * self.Vd)
        self.w_in = self.wo = self.b_in = self.w_qnorm = self.w_knorm = None
        self.inv_freq = self.inv_freq_v = None
        self.rot = 0
        self.rot_magnitude = 1.0
        self.lam = 0.0

    # ------------------------------------------------------------------ tensors
    def params(self):
        d, H, G, D, Vd, m = self.d, self.H, self.G, self.D, self.Vd, self.maps
        p = {"q_proj": ParamSpec((H * m * D, d)), "k_proj": ParamSpec((G * m * D, d)), "o_proj": ParamSpec((d, H * Vd))}
        if not self.values_from_keys:
            p["v_proj"] = ParamSpec((G * Vd, d))
        if self.taps:
            p.update({"q_conv": ParamSpec((H * D, self.taps), kind="vector", init="normal"),
                      "k_conv": ParamSpec((G * D, self.taps), kind="vector", init="normal")})
        if self.head_norm:
            p.update({"q_norm": ParamSpec((D,), kind="vector", init="ones"), "k_norm": ParamSpec((D,), kind="vector", init="ones")})
        if self.bias:
            p.update({"q_bias": ParamSpec((H * m * D,), kind="vector", init="normal"),
                      "k_bias": ParamSpec((G * m * D,), kind="vector", init="normal"),
                      "v_bias": ParamSpec((G * Vd,), kind="vector", init="normal")})
        if self.projection_norm:
            p.update({"q_norm": ParamSpec((H * D,), kind="vector", init="ones"),
                      "k_norm": ParamSpec((G * D,), kind="vector", init="ones")})
        if self.maps == 2:
            p.update({k: ParamSpec((D,), kind="vector", init="normal") for k in ("lambda_q1", "lambda_k1", "lambda_q2", "lambda_k2")})
        if self.head_gate:
            p["gate_proj"] = ParamSpec((H, d))
        if self.sinks and not self.zero_sinks:
            p["sink"] = ParamSpec((H,), kind="vector", init="normal")
        return p

    def _by_map(self, t, heads):
        """Rows [head][map][D] of a projection (or bias) reordered to [map][head][D]."""
        if self.maps == 1:
            return t
        rest = t.shape[1:]
        return t.reshape(heads, self.maps, self.D, *rest).transpose(0, 1).reshape(heads * self.maps * self.D, *rest).contiguous()

    def load(self, t):
        H, G = self.H, self.G
        mats = [self._by_map(t["q_proj"], H), self._by_map(t["k_proj"], G)] + ([] if self.values_from_keys else [t["v_proj"]])
        if self.head_gate:
            mats.append(t["gate_proj"])
        dts = {m.dtype for m in mats}
        dt = torch.float32 if len(dts) > 1 else dts.pop()
        w = torch.cat([m.to(dt) for m in mats], dim=0)
        pad = -w.shape[0] % 16           # whole bands of 16 rows: the weight can be kept in operand order
        if pad:
            w = torch.cat([w, torch.zeros((pad, w.shape[1]), dtype=dt, device=w.device)], dim=0)
        self.n_in = w.shape[0]
        self.w_in = Weight(w)
        self.wo = Weight(t["o_proj"])
        if self.bias:
            self.b_in = torch.cat([self._by_map(t["q_bias"], H), self._by_map(t["k_bias"], G), t["v_bias"]]).float().contiguous()
        if self.projection_norm or self.head_norm:
            self.w_qnorm, self.w_knorm = t["q_norm"].float().contiguous(), t["k_norm"].float().contiguous()
        if self.taps:
            # tap by tap, [taps, channels]: the kernel's loads of one tap are consecutive
            self.w_conv = torch.cat([t["q_conv"].float(), t["k_conv"].float()], dim=0).t().contiguous()
        if self.score_position is not None:
            self.slopes = self.score_position.score_slopes(self.HQ)
        if self.maps == 2:
            dot = lambda a, b: float((t[a].double() * t[b].double()).sum())
            self.lam = math.exp(dot("lambda_q1", "lambda_k1")) - math.exp(dot("lambda_q2", "lambda_k2")) + self.diff
        if self.sinks:
            self.w_sink = torch.zeros(H, dtype=torch.float32, device=self.env.device) if self.zero_sinks \
                else t["sink"].float().contiguous()
        if self.position is not None:
            ka = self.position.kernel_args()
            if ka["use_rope"]:
                self.inv_freq, self.rot = ka["inv_freq"], int(ka.get("rotary_dim") or self.D)
                self.rot_magnitude = float(ka.get("magnitude", 1.0))
                if self.rot > self.D:
                    raise ValueError(f"wide_attention: {self.rot} turning elements in heads of {self.D}")
        if self.value_position is not None:
            ka = self.value_position.kernel_args()
            if int(ka.get("rotary_dim") or self.Vd) != self.Vd or self.Vd % 2 or ka.get("magnitude", 1.0) != 1.0:
                raise ValueError("wide_attention: the values' rotation is a pure one over the whole (even) value width")
            self.inv_freq_v = ka["inv_freq"]

    def slow_paths(self, page_size):
        notes = []
        if self.env.dtype == torch.bfloat16:
            if not self._mfma(page_size):
                notes.append(f"attention runs on plain FMAs: keys of {self.D} and values of {self.Vd} elements, pages of "
                             f"{page_size} (the MFMA kernels take values of 64 or 128 with keys no wider, at most 16 query heads "
                             f"a kv head, and pages in multiples of 32)")
            for name, w in (("q/k/v projection", self.w_in), ("output projection", self.wo)):
                if w is not None:
                    notes += w.slow_reason(name)
        return notes

    def cache_need(self):
        from .base import StateNeed
        # with a convolution: the last taps - 1 projected q and k rows of the request, fp32
        state = StateNeed((self.taps - 1, self.n_qk), torch.float32) if self.taps > 1 else None
        return CacheNeed(kv=KVNeed(self.GK, self.Dk, self.visibility, self.span, v_head_dim=self.Vd, n_v_heads=self.G),
                         state=state)

    def _mfma(self, page_size):
        return (self.env.dtype == torch.bfloat16 and self.Dk == self.Vd and self.Vd in (64, 128) and page_size % 32 == 0
                and self.HQ // self.GK <= 16)

    # ------------------------------------------------------------------ the step
    def _decode(self, q, o, ctx, cache, T):
        HQ, GK, D = self.HQ, self.GK, self.Dk
        longest = cache.block_table.shape[1] * cache.page_size
        if self.visibility != "full":
            longest = min(longest, self.span + 32)
        blocks = -(-longest // 32)
        n_splits = max(1, min(-(-2 * hipops.cu_count() // (T * GK)), -(-blocks // 8), 256))
        scratch = ctx.ws.take((hipops.attn_decode_workspace(T, HQ, D, n_splits) // 4,), torch.float32)
        hipops.attn_decode(q, cache.k_pages, cache.v_pages, o, scratch, ctx.positions, ctx.seq_of_token,
                           cache.block_table, T, HQ, GK, D, cache.page_size, self.visibility, self.span,
                           self.scale, n_splits, value_heads=self.G, sinks=self.w_sink, slopes=self.slopes)

    def _prefill(self, q, o, ctx, cache, lead, cu_seqlens):
        HQ, GK, D = self.HQ, self.GK, self.Dk
        counts, starts = ctx.host.counts[lead:], ctx.host.starts[lead:]
        longest = int((starts + counts).max())
        if self.visibility != "full":
            longest = min(longest, self.span + int(counts.max()))
        n_splits = hipops.attn_prefill_splits(counts, HQ, GK, longest)
        scratch = None
        if n_splits > 1:
            scratch = ctx.ws.take((hipops.attn_prefill_workspace(counts, HQ, GK, D, n_splits) // 4,), torch.float32)
        hipops.attn_prefill(q, cache.k_pages, cache.v_pages, o, ctx.positions[lead:], cu_seqlens, counts,
                            cache.block_table[lead:], HQ, GK, D, cache.page_size, self.visibility, self.span, self.scale,
                            n_splits=n_splits, scratch=scratch, value_heads=self.G, sinks=self.w_sink, slopes=self.slopes)

    def forward(self, x, ctx, cache):
        T, ws = x.shape[0], ctx.ws
        H, G, HQ, GK, D, Vd, Dk = self.H, self.G, self.HQ, self.GK, self.D, self.Vd, self.Dk
        proj = ws.take((T, self.n_in), x.dtype)
        linear(x, self.w_in, proj, ws=ws)
        conv = None
        if self.taps:
            # (with values taken from the keys the convolved rows are all that the next kernel reads)
            conv = ws.take((T, self.n_qk), x.dtype)
            hipops.causal_conv(proj[:, :self.n_qk], self.w_conv, conv, cache.state, ctx.seq_of_token, ctx.cu_seqlens,
                               ctx.seq_slots, keep=cache.write)
        q = ws.take((T, HQ * Dk), x.dtype)
        hipops.qkv_prepare(conv if self.taps else proj, q, cache.k_pages, cache.v_pages, ctx.positions, cache.slot_map, HQ, GK, G, D, Vd,
                           cache.page_size, bias=self.b_in, norm_q=self.w_qnorm, norm_k=self.w_knorm, eps=self.eps,
                           inv_freq=self.inv_freq, rot=self.rot, inv_freq_v=self.inv_freq_v, write_kv=cache.write,
                           k_tiled=cache.tiled, v_tiled=cache.tiled, stored_dim=Dk, rot_magnitude=self.rot_magnitude,
                           head_norm=self.head_norm, q_temperature=self.q_temperature, values_from_keys=self.values_from_keys)
        if cache.tiled and self._mfma(cache.page_size):
            a = ws.take((T, HQ * Vd), x.dtype)
            cu_tail, lead = ctx.derived[TAIL]
            if ctx.decode_only:
                self._decode(q, a, ctx, cache, T)
            else:
                if lead:                   # decoded tokens of other requests beside prompt portions
                    self._decode(q, a, ctx, cache, lead)
                self._prefill(q[lead:], a[lead:], ctx, cache, lead, cu_tail if lead else ctx.cu_seqlens)
        else:
            # two maps meet in a difference: keep them in fp32 until then
            a = ws.take((T, HQ * Vd), torch.float32 if self.maps == 2 else x.dtype)
            hipops.attn_wide(q, cache.k_pages, cache.v_pages, a, ctx.positions, ctx.seq_of_token, cache.block_table,
                             T, HQ, GK, G, Dk, Vd, cache.page_size, self.visibility, self.span, self.scale,
                             k_tiled=cache.tiled, v_tiled=cache.tiled, sinks=self.w_sink, slopes=self.slopes)
        if self.maps == 2 or self.inv_freq_v is not None or self.head_gate:
            o = ws.take((T, H * Vd), x.dtype)
            gate = proj[:, self.n_qkv:self.n_qkv + H] if self.head_gate else None
            hipops.attn_finish(a, o, ctx.positions, H, Vd, maps=self.maps, lam=self.lam, eps=self.eps,
                               post=1.0 - self.diff, inv_freq_v=self.inv_freq_v, gate=gate)
        else:
            o = a
        out = ws.take((T, self.d), torch.float32)
        linear(o, self.wo, out, ws=ws)
        return out
