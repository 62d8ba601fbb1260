"""The two ends of a model: token ids in, logits out.

``token_table`` (crates/spite-models/src/llama/llama4.rs:118-119): row ``id`` of the table as
the residual stream's first value, in fp32, times ``scale`` if the architecture has one.
``linear_head`` (llama4.rs:277-279): logits = W . (normed last hidden state), W ``[V, d]``;
tied, it reads the embedding's table; times ``scale`` if the architecture has one; with ``softcap`` c the
logits become c * tanh(logits / c).  Another architecture's embedding scale, logit cap or
bias is another kind registered under these categories, not a change to the model class.

``token_pair_table``: the token's row plus a row of a second table chosen by a hash of the token and the one
before it, (previous * mul_prev + token * mul_cur) mod buckets; a request's first token takes the table's last
row (number ``buckets``).  The previous token of a request is its state between steps.
"""
from __future__ import annotations

import torch

from .base import Embedding, Head, ParamSpec, StateNeed, register
from .linear import linear, Weight
from ..csrc import hipops


@register("embedding", "token_table")
class TokenTable(Embedding):
    graph_safe = True

    def __init__(self, env, vocab_size: int, width: int, scale: float = 1.0):
        """``scale``: a constant on every row as it enters the stream (fp32)."""
        self.V, self.d, self.scale = int(vocab_size), int(width), float(scale)
        self.table = None

    def params(self):
        return {"weight": ParamSpec((self.V, self.d))}

    def load(self, tensors):
        self.table = tensors["weight"].contiguous()

    def forward(self, token_ids, h, ctx, state=None):
        hipops.embed(token_ids, self.table, h, self.scale)


@register("embedding", "token_pair_table")
class TokenPairTable(Embedding):
    graph_safe = True

    def __init__(self, env, vocab_size: int, width: int, buckets: int, mul_prev: int, mul_cur: int, scale: float = 1.0):
        self.V, self.d, self.scale = int(vocab_size), int(width), float(scale)
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        if self.buckets < 1:
            raise ValueError(f"token_pair_table: {buckets} buckets")
        self.table = self.pairs = None

    def params(self):
        return {"weight": ParamSpec((self.V, self.d)), "pairs": ParamSpec((self.buckets + 1, self.d))}

    def load(self, tensors):
        self.table = tensors["weight"].contiguous()
        self.pairs = tensors["pairs"].to(self.table.dtype).contiguous()

    def state_need(self):
        return StateNeed((), torch.int32)

    def forward(self, token_ids, h, ctx, state=None):
        if state is None:
            raise ValueError("token_pair_table: the model spec gives the embedding no cache id for its state")
        rows = ctx.ws.take((h.shape[0],), torch.int32)
        hipops.hash_rows(token_ids, ctx.positions, ctx.seq_of_token, ctx.cu_seqlens, ctx.seq_slots, state, rows,
                         self.mul_prev, self.mul_cur, self.buckets)
        hipops.embed_sum(token_ids, self.table, rows, self.pairs, h, self.scale)


@register("head", "linear_head")
class LinearHead(Head):
    graph_safe = True

    def __init__(self, env, vocab_size: int, width: int, tied: bool = False, scale: float = 1.0, softcap: float = 0.0):
        """``scale``: a constant on the logits (fp32); ``softcap`` c > 0: logits = c * tanh(logits / c) after it."""
        self.V, self.d, self.tied, self.scale = int(vocab_size), int(width), bool(tied), float(scale)
        self.softcap = float(softcap or 0.0)
        self.weight = None

    def params(self):
        return {} if self.tied else {"weight": ParamSpec((self.V, self.d))}

    def load(self, tensors):
        if not self.tied:
            self.weight = Weight(tensors["weight"])

    def tie(self, embedding):
        """Tied: the table stays row-major (the embedding reads its rows) and serves as W."""
        if self.tied:
            self.weight = embedding.table

    def slow_paths(self, page_size):
        return self.weight.slow_reason("output matrix") if isinstance(self.weight, Weight) else []

    def forward(self, x, logits, ctx):
        linear(x, self.weight, logits, ws=ctx.ws)
        if self.scale != 1.0:
            hipops.scale_rows(logits, self.scale)
        if self.softcap > 0.0:
            hipops.softcap_rows(logits, self.softcap)
