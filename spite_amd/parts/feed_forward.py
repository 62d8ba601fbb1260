"""Feed-forward parts.

``dense_glu`` (crates/spite-models/src/llama/llama4.rs:257-271):
y = W_down . (act(W_gate . x) * (W_up . x)), act = silu there; ``gelu_tanh`` and ``relu`` are the
gate's other activations.

``dense_mlp``: y = W_down . act(W_up . x), no gate; ``activation``: ``gelu`` (the erf form),
``gelu_tanh`` or ``silu``, applied in fp32 to the up projection's rows.

``moe_top1_sigmoid`` (crates/spite-models/src/moe.rs:87-194, llama4.rs:212-256): router
logits W_r . x in fp32; the expert with the largest logit (lowest index on ties); its
*input* is x * sigmoid(logit), its output is not weighted; a shared expert on the unscaled
x is added.  Routed and shared experts run as one grouped product over a row list: group
e < E holds the tokens routed to expert e, group E every token (at 33 to 64 tokens the shared
expert's group runs as a plain product of its own over the same rows).

``moe_topk_sigmoid``: router logits in fp32; scores s = sigmoid(logit); the ``top_k`` experts with
the largest s + bias (a per-expert correction that steers the choice only); each taken expert's
*output* is weighted with its s (divided by the taken scores' sum if ``renormalize``); a shared
expert of its own width may run for every token.  The choices of a step are ``top_k`` entries a
token; the expert plan sorts them by expert, the grouped products walk that list, every entry
gets an output row of its own and a last kernel forms the weighted sum per token.

With ``weight_input`` the weight multiplies the expert's input instead (the grouped product scales the rows it
reads) and the outputs are summed as they are.

``moe_topk_softmax``: the same part with the other way of scoring: the ``top_k`` experts with the largest
logits are taken and their weights are the softmax over the taken logits alone; no bias.
"""
from __future__ import annotations

import math

import torch

from .base import FeedForward, ParamSpec, register
from .linear import SKINNY_MAX_ROWS, Weight, grouped_tile_shape, linear
from ..csrc import hipops


@register("ffn", "dense_glu")
class DenseGLU(FeedForward):
    graph_safe = True

    def __init__(self, env, hidden_size, intermediate_size, activation="silu"):
        """``activation``: the gate's, ``silu``, ``gelu_tanh`` or ``relu``."""
        self.d, self.F = int(hidden_size), int(intermediate_size)
        if hipops.GATE_ACTS.get(activation, 0) == 0:
            raise ValueError(f"dense_glu: activation {activation!r} (known: silu, gelu_tanh, relu)")
        self.activation = activation
        self.w_gate_up = self.w_down = None

    def params(self):
        return {"gate_proj": ParamSpec((self.F, self.d)), "up_proj": ParamSpec((self.F, self.d)),
                "down_proj": ParamSpec((self.d, self.F))}

    def load(self, t):
        dt = t["gate_proj"].dtype if t["gate_proj"].dtype == t["up_proj"].dtype else torch.float32
        # gate rows then up rows: the up row of a gate row lies F rows further on; in operand order
        # that needs whole bands, F a multiple of 16
        self.w_gate_up = Weight(torch.cat([t["gate_proj"].to(dt), t["up_proj"].to(dt)], dim=0), self.F % 16 == 0)
        self.w_down = Weight(t["down_proj"])

    def slow_paths(self, page_size):
        return self.w_gate_up.slow_reason("gate/up projection") + self.w_down.slow_reason("down projection")

    def forward(self, x, x32, ctx, projected=None):
        T = x.shape[0]
        act = ctx.ws.take((T, self.F), x.dtype)
        linear(x, self.w_gate_up, act, glu=self.activation, ws=ctx.ws)
        y = ctx.ws.take((T, self.d), torch.float32)
        linear(act, self.w_down, y, ws=ctx.ws)
        return (y,)


@register("ffn", "dense_mlp")
class DenseMLP(FeedForward):
    graph_safe = True

    def __init__(self, env, hidden_size, intermediate_size, activation="gelu"):
        self.d, self.F = int(hidden_size), int(intermediate_size)
        if activation not in hipops.UNARY_ACTS:
            raise ValueError(f"dense_mlp: activation {activation!r} (known: {sorted(hipops.UNARY_ACTS)})")
        self.activation = activation
        self.w_up = self.w_down = None

    def params(self):
        return {"up_proj": ParamSpec((self.F, self.d)), "down_proj": ParamSpec((self.d, self.F))}

    def load(self, t):
        self.w_up, self.w_down = Weight(t["up_proj"]), Weight(t["down_proj"])

    def slow_paths(self, page_size):
        return self.w_up.slow_reason("up projection") + self.w_down.slow_reason("down projection")

    def forward(self, x, x32, ctx, projected=None):
        T = x.shape[0]
        u = ctx.ws.take((T, self.F), x.dtype)
        linear(x, self.w_up, u, ws=ctx.ws, act=self.activation)
        y = ctx.ws.take((T, self.d), torch.float32)
        linear(u, self.w_down, y, ws=ctx.ws)
        return (y,)


@register("ffn", "moe_top1_sigmoid")
class MoeTop1Sigmoid(FeedForward):
    graph_safe = True

    wants_f32_input = True

    def __init__(self, env, hidden_size, intermediate_size, n_experts, shared_intermediate_size=None):
        self.d, self.F, self.E = int(hidden_size), int(intermediate_size), int(n_experts)
        self.Fs = int(shared_intermediate_size if shared_intermediate_size is not None else intermediate_size)
        if self.E < 1 or self.E > 65000:
            raise ValueError(f"moe: {self.E} experts")
        self.fused_shared = self.Fs == self.F
        self.w_router = self.w_gate_up = self.w_down = None
        self.ws_gate_up = self.ws_down = None

    def params(self):
        d, F, Fs, E = self.d, self.F, self.Fs, self.E
        return {"router": ParamSpec((E, d), kind="vector"),
                "experts.gate_up_proj": ParamSpec((E, d, 2 * F)), "experts.down_proj": ParamSpec((E, F, d)),
                "shared.gate_proj": ParamSpec((Fs, d)), "shared.up_proj": ParamSpec((Fs, d)),
                "shared.down_proj": ParamSpec((d, Fs))}

    def load(self, t):
        self.w_router = t["router"].contiguous()
        # checkpoint [E, d, 2F] (x @ M) -> [E, 2F, d] rows of gate then up; down [E, F, d] -> [E, d, F]
        gu = t["experts.gate_up_proj"].transpose(1, 2)
        dn = t["experts.down_proj"].transpose(1, 2)
        sgu = torch.cat([t["shared.gate_proj"], t["shared.up_proj"]], dim=0)
        sdn = t["shared.down_proj"]
        if self.fused_shared and sgu.dtype == gu.dtype and sdn.dtype == dn.dtype:
            self.w_gate_up = Weight(torch.cat([gu, sgu[None]], dim=0), self.F % 16 == 0)
            self.w_down = Weight(torch.cat([dn, sdn[None]], dim=0))
        else:
            self.fused_shared = False
            self.w_gate_up, self.w_down = Weight(gu, self.F % 16 == 0), Weight(dn)
            self.ws_gate_up, self.ws_down = Weight(sgu, self.Fs % 16 == 0), Weight(sdn)

    def slow_paths(self, page_size):
        ws = [("experts' gate/up", self.w_gate_up), ("experts' down", self.w_down),
              ("shared expert's gate/up", self.ws_gate_up), ("shared expert's down", self.ws_down)]
        return [n for name, w in ws if w is not None for n in w.slow_reason(name)]

    def _few_rows_a_group(self, T: int) -> bool:
        """Whether a routed group of a step of T tokens is unlikely to hold more than 16 rows
        (group sizes taken as normal around T/E: mean + 4 sd)."""
        mean = T / self.E
        return mean + 4.0 * math.sqrt(T * (1.0 / self.E) * (1.0 - 1.0 / self.E)) <= 16.0

    def input_projection(self):
        return self.w_router if self.w_router is not None and self.w_router.dtype == torch.float32 else None

    def forward(self, x, x32, ctx, projected=None):
        """``projected``: the router's logits [T, E] if the block's norm formed them; else they
        are computed here from x32."""
        T, E, F, d = x.shape[0], self.E, self.F, self.d
        ws = ctx.ws
        expert = ws.take((T,), torch.int32)
        weight = ws.take((T,), torch.float32)
        trace = ctx.extras.get("trace")
        if trace is not None and trace.get("take_experts"):
            # a testing aid: the experts are given (one tensor per call, in the order of the
            # calls), each with the weight that its own logit gives; every other logit is
            # taken out before the plan is made
            take = trace["take_experts"].pop(0).to(device=x.device, dtype=torch.int64).view(T, 1)
            logits = projected
            if logits is None:
                logits = ws.take((T, E), torch.float32)
                hipops.gemm_generic(x32, self.w_router, logits, T, E, d)
            projected = torch.full_like(logits, float("-inf")).scatter_(1, take, logits.gather(1, take))
        if projected is None:
            hipops.router_top1(x32, self.w_router, expert, weight)
        n = 2 * T if self.fused_shared else T
        src, dst = ws.take((n,), torch.int32), ws.take((n,), torch.int32)
        scale = ws.take((n,), torch.float32)
        groups = E + 1 if self.fused_shared else E
        offsets = ws.take((groups + 1,), torch.int32)
        hipops.moe_plan(expert, weight, src, scale, dst, offsets, T, E, self.fused_shared, logits=projected)
        if trace is not None:                         # a testing aid: which expert each row took
            trace.setdefault("moe_experts", []).append(expert.clone())
        act = ws.take((n, F), x.dtype)
        y = ws.take((2 * T, d), torch.float32)
        if self.fused_shared and self.w_gate_up.tiled and 32 < T <= SKINNY_MAX_ROWS and self._few_rows_a_group(T):
            # 33 to 64 tokens: the routed groups hold a few rows each and take the weight stream's
            # narrow form (16 token columns); the shared expert, which takes every row, would be
            # read once per 16 of them there, so it runs as a plain product of its own (measured
            # at 64 tokens over 16 experts: 658 against 683 us for the two products of a layer)
            linear(x, self.w_gate_up, act, glu=True, offsets=offsets, n_groups=E, a_rows=src, a_scale=scale, rows=T,
                   max_rows=16, ws=ws)
            linear(x, self.w_gate_up.group(E), act[T:], glu=True, a_rows=src[T:], a_scale=scale[T:], rows=T, ws=ws)
            linear(act, self.w_down, y, offsets=offsets, n_groups=E, y_rows=dst, rows=T, max_rows=16, ws=ws)
            linear(act[T:], self.w_down.group(E), y, y_rows=dst[T:], rows=T, ws=ws)
            return (y[:T], y[T:])
        # the tile of either product, by the rounds that its tiles make on the chip (gate and up
        # rows share a tile of 512 W rows: 256 columns of the result; the down product's tile has 512)
        shape = grouped_tile_shape(T, E, groups - E, col_tiles=-(-F // 256)) if T > SKINNY_MAX_ROWS else 0
        shape_down = grouped_tile_shape(T, E, groups - E, col_tiles=-(-d // 512)) if T > SKINNY_MAX_ROWS else 0
        # every token goes to one expert: at most min(T, E) of their groups hold rows, and the shared one
        live = min(T, E) + (groups - E)
        linear(x, self.w_gate_up, act, glu=True, offsets=offsets, n_groups=groups, a_rows=src, a_scale=scale, rows=n,
               max_rows=T, tile_shape=shape, live_groups=live, ws=ws)
        # slot s writes row dst[s]: rows [0,T) the routed result per token, rows [T,2T) the shared one
        linear(act, self.w_down, y, offsets=offsets, n_groups=groups, y_rows=dst, rows=n, max_rows=T,
               tile_shape=shape_down, live_groups=live, ws=ws)
        if self.fused_shared:
            return (y[:T], y[T:])
        act_s = ws.take((T, self.Fs), x.dtype)
        linear(x, self.ws_gate_up, act_s, glu=True, ws=ws)
        linear(act_s, self.ws_down, y[T:], ws=ws)
        return (y[:T], y[T:])


@register("ffn", "moe_topk_sigmoid")
class MoeTopKSigmoid(FeedForward):
    graph_safe = True
    wants_f32_input = True

    def __init__(self, env, hidden_size, intermediate_size, n_experts, top_k, shared_intermediate_size=None,
                 score_bias=True, renormalize=False, activation="silu", scoring="sigmoid", weight_input=False):
        """``scoring``: ``sigmoid`` (the choice by sigmoid(z) + bias, weights sigmoid(z)) or ``softmax_taken`` (the
        choice by z + bias, weights the softmax over the taken experts' z).  ``weight_input``: the weight multiplies
        the expert's input instead of its output: the result is the sum of expert(w * x)."""
        self.weight_input = bool(weight_input)
        if scoring not in hipops.ROUTER_SCORING:
            raise ValueError(f"moe: scoring {scoring!r} (known: {sorted(hipops.ROUTER_SCORING)})")
        self.scoring = scoring
        self.d, self.F, self.E, self.k = int(hidden_size), int(intermediate_size), int(n_experts), int(top_k)
        self.Fs = None if shared_intermediate_size is None else int(shared_intermediate_size)
        if not 1 <= self.k <= self.E or self.E > 512:
            raise ValueError(f"moe: {self.k} of {self.E} experts (at most 512)")
        if hipops.GATE_ACTS.get(activation, 0) == 0:
            raise ValueError(f"moe: activation {activation!r} (known: silu, gelu_tanh, relu)")
        self.score_bias, self.renormalize, self.activation = bool(score_bias), bool(renormalize), activation
        self.w_router = self.bias = self.w_gate_up = self.w_down = self.ws_gate_up = self.ws_down = None

    def params(self):
        d, F, E = self.d, self.F, self.E
        p = {"router": ParamSpec((E, d), kind="vector")}
        if self.score_bias:
            p["correction"] = ParamSpec((E,), kind="vector", init="normal")
        for e in range(E):
            p[f"e{e}.gate"], p[f"e{e}.up"], p[f"e{e}.down"] = ParamSpec((F, d)), ParamSpec((F, d)), ParamSpec((d, F))
        if self.Fs is not None:
            p["shared.gate"], p["shared.up"] = ParamSpec((self.Fs, d)), ParamSpec((self.Fs, d))
            p["shared.down"] = ParamSpec((d, self.Fs))
        return p

    def load(self, t):
        E = self.E
        self.w_router = t["router"].contiguous()
        self.bias = t["correction"].contiguous() if self.score_bias else None
        dts = {t[f"e{e}.{k}"].dtype for e in range(E) for k in ("gate", "up", "down")}
        dt = torch.float32 if len(dts) > 1 else dts.pop()
        gu = torch.stack([torch.cat([t[f"e{e}.gate"].to(dt), t[f"e{e}.up"].to(dt)], dim=0) for e in range(E)])
        self.w_gate_up = Weight(gu, self.F % 16 == 0)
        del gu
        self.w_down = Weight(torch.stack([t[f"e{e}.down"].to(dt) for e in range(E)]))
        if self.Fs is not None:
            sdt = t["shared.gate"].dtype if t["shared.gate"].dtype == t["shared.up"].dtype else torch.float32
            self.ws_gate_up = Weight(torch.cat([t["shared.gate"].to(sdt), t["shared.up"].to(sdt)], dim=0), self.Fs % 16 == 0)
            self.ws_down = Weight(t["shared.down"])

    def slow_paths(self, page_size):
        ws = [("experts' gate/up", self.w_gate_up), ("experts' down", self.w_down),
              ("shared expert's gate/up", self.ws_gate_up), ("shared expert's down", self.ws_down)]
        return [n for name, w in ws if w is not None for n in w.slow_reason(name)]

    def input_projection(self):
        return self.w_router if self.w_router is not None and self.w_router.dtype == torch.float32 else None

    def forward(self, x, x32, ctx, projected=None):
        T, E, F, d, k = x.shape[0], self.E, self.F, self.d, self.k
        ws = ctx.ws
        logits = projected
        if logits is None:
            logits = ws.take((T, E), torch.float32)
            hipops.gemm_generic(x32, self.w_router, logits, T, E, d)
        n = T * k
        expert, weight = ws.take((n,), torch.int32), ws.take((n,), torch.float32)
        trace = ctx.extras.get("trace")
        bias = self.bias
        if trace is not None and trace.get("take_experts"):
            # a testing aid: the experts are given ([T, top_k] per call, in the order of the calls), each
            # with the weight that its own logit gives; every other logit is taken out of the choice
            take = trace["take_experts"].pop(0).to(device=x.device, dtype=torch.int64).view(T, k)
            logits = torch.full_like(logits, float("-inf")).scatter_(1, take, logits.gather(1, take))
            bias = None
        hipops.router_topk(logits, bias, expert, weight, k, renorm=self.renormalize, scoring=self.scoring)
        if trace is not None:                         # a testing aid: which experts each token took, [T, top_k]
            trace.setdefault("moe_experts", []).append(expert.view(T, k).clone())
        # (``unused``: the entries' weights in the order of the slots; a product reads it only with ``weight_input``)
        src, dst, unused = ws.take((n,), torch.int32), ws.take((n,), torch.int32), ws.take((n,), torch.float32)
        offsets = ws.take((E + 1,), torch.int32)
        hipops.moe_plan(expert, weight, src, unused, dst, offsets, n, E, False, fan=k)
        live = min(n, E)
        # slot s (entries sorted by expert) reads token src[s] and writes the entry's own row dst[s]
        act = ws.take((n, F), x.dtype)
        linear(x, self.w_gate_up, act, glu=self.activation, offsets=offsets, n_groups=E, a_rows=src,
               a_scale=unused if self.weight_input else None, rows=n, max_rows=T, live_groups=live, ws=ws)
        y = ws.take((n, d), torch.float32)
        linear(act, self.w_down, y, offsets=offsets, n_groups=E, y_rows=dst, rows=n, max_rows=T, live_groups=live, ws=ws)
        ys = None
        if self.Fs is not None:
            act_s = ws.take((T, self.Fs), x.dtype)
            linear(x, self.ws_gate_up, act_s, glu=self.activation, ws=ws)
            ys = ws.take((T, d), torch.float32)
            linear(act_s, self.ws_down, ys, ws=ws)
        out = ws.take((T, d), torch.float32)
        hipops.moe_combine(y, None if self.weight_input else weight, ys, out, T, k)
        return (out,)


@register("ffn", "moe_topk_softmax")
class MoeTopKSoftmax(MoeTopKSigmoid):
    """Several experts a token, taken by their logits and weighted by the softmax over the taken ones."""

    def __init__(self, env, hidden_size, intermediate_size, n_experts, top_k, shared_intermediate_size=None,
                 activation="silu"):
        super().__init__(env, hidden_size, intermediate_size, n_experts, top_k, shared_intermediate_size,
                         score_bias=False, renormalize=False, activation=activation, scoring="softmax_taken")
