"""A Nolapel model as a list of parts.

Every layer is a ``sandwich`` block with tanh norms before and after each sublayer.  Mixers: ``attention`` is
``wide_attention`` with a convolution on q and k, a head norm, a query temperature, distance slopes, a window, a sink
of score zero and values taken from the keys; ``parallel`` is a ``mixer_sum`` of ``wide_attention`` (rotation of a
head's leading part, learned sinks, every earlier key) and ``time_mix``; ``mamba2`` is ``state_space``.  Feed-forward:
``moe_topk_sigmoid`` with the weight on the expert's input, no choice bias and a shared expert.  The embedding is a
``token_pair_table`` where the model has the hashed second table; the logits pass a soft cap.  A looped run of layers
is the same blocks called once per pass, each pass with cache ids of its own, with a ``reentry`` call before each.
Tensor names: ``l<i>.norm1|norm1b|norm2|norm2b`` (+ ``.b``, ``.alpha``), ``.mix.*``, ``.mlp.router|e<k>.*|shared.*``;
``embed``, ``bigram``, ``loop.in``, ``loop.step``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from .nolapel import NolapelConfig
from .registry import register_architecture
from ..parts.base import PartSpec, BlockSpec, LayerCall, ModelSpec


def _tanh_norm(d, name):
    return PartSpec("tanh", {"width": d}, {"weight": name, "bias": name + ".b", "alpha": name + ".alpha"})


def _attention(d, a, p, eps, plain):
    """``plain``: the 'attention' kind (values are keys); else the rotated kind with learned sinks."""
    names = {"q_proj": p + "q", "k_proj": p + "k", "o_proj": p + "o"}
    args = dict(hidden_size=d, n_heads=a.heads, n_kv_heads=a.kv_heads, key_dim=a.dim, value_dim=a.vdim, scale=a.scale,
                visibility="full" if a.window is None else "window", span=a.window or 0, norm_eps=eps)
    if plain:
        names.update({"q_norm": p + "q.norm", "k_norm": p + "k.norm"})
        args.update(head_norm=True, values="keys", sinks="zero", q_temperature=a.q_temp,
                    score_position=PartSpec("distance_slopes", {"ratio": 8.0}))
        if a.conv >= 1:
            names.update({"q_conv": p + "q.conv", "k_conv": p + "k.conv"})
            args.update(conv_taps=a.conv)
    else:
        names.update({"v_proj": p + "v", "sink": p + "sink"})
        position = None
        if a.rot_base is not None and a.rot_dims > 0:
            position = PartSpec("rotary", {"head_dim": a.dim, "theta": a.rot_base, "rotary_dim": a.rot_dims})
        args.update(position=position, sinks=True)
    return PartSpec("wide_attention", args, names)


def _mixer(d, layer, p, eps):
    mx = layer.mixer
    if layer.type == "attention":
        return _attention(d, mx, p, eps, plain=True)
    if layer.type == "parallel":
        left, right, ls, rs = mx
        la = _attention(d, left, p + "left.", eps, plain=False)
        r = p + "right."
        names = {f"mu_{s}": f"{r}mu.{s}" for s in "rkvgw"}
        names.update({f"{s}_proj": r + s for s in "rkvg"})
        names.update({"decay_down": r + "w1", "decay_up": r + "w2", "decay_bias": r + "w0", "bonus": r + "u",
                      "norm": r + "norm", "o_proj": r + "o"})
        ra = PartSpec("time_mix", dict(hidden_size=d, n_heads=right.heads, head_dim=right.dim, norm_eps=eps), names)
        both = {f"left.{k}": v for k, v in la.names.items()}
        both.update({f"right.{k}": v for k, v in ra.names.items()})
        return PartSpec("mixer_sum", {"parts": {"left": la, "right": ra}, "scales": {"left": ls, "right": rs}}, both)
    names = {"in_proj": p + "in", "conv": p + "conv", "conv_bias": p + "conv.b", "dt_bias": p + "dt_bias", "a_log": p + "A_log",
             "skip": p + "D", "norm": p + "norm", "o_proj": p + "o"}
    return PartSpec("state_space", dict(hidden_size=d, n_heads=mx.heads, value_dim=mx.vdim, state_dim=mx.state, n_groups=mx.groups,
                                        conv_taps=mx.conv, norm_groups=mx.norm_groups, norm_eps=eps), names)


def _cache_names(layer):
    """The names that a layer's block gives its caches (what ``Block.cache_needs`` will return)."""
    if layer.type == "attention":
        return [""]
    if layer.type == "parallel":
        return ["left", "right.state", "right.shift"]
    return ["state"] + (["conv"] if layer.mixer.conv > 1 else [])


def build_spec(cfg: NolapelConfig) -> ModelSpec:
    d, eps = cfg.width, cfg.norm_eps
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        ffn = None
        if layer.mlp is not None:
            ml, f = layer.mlp, p + "mlp."
            fn = {"router": f + "router"}
            for e in range(ml.experts):
                fn.update({f"e{e}.{k}": f"{f}e{e}.{k}" for k in ("gate", "up", "down")})
            if ml.shared_ff is not None:
                fn.update({f"shared.{k}": f"{f}shared.{k}" for k in ("gate", "up", "down")})
            ffn = PartSpec("moe_topk_sigmoid", dict(
                hidden_size=d, intermediate_size=ml.expert_ff, n_experts=ml.experts, top_k=ml.top,
                shared_intermediate_size=ml.shared_ff, score_bias=False, renormalize=False, activation="silu",
                weight_input=True), fn)
        extra = {"norm1b": _tanh_norm(d, p + "norm1b"), "residual_mult": 1.0}
        if ffn is not None:
            extra["norm2b"] = _tanh_norm(d, p + "norm2b")
        blocks.append(BlockSpec("sandwich", _tanh_norm(d, p + "norm1"), _mixer(d, layer, p + "mix.", eps),
                                _tanh_norm(d, p + "norm2") if ffn is not None else None, ffn, extra))
    n_layers = len(cfg.layers)
    next_id = [0]

    def call(i):
        names = _cache_names(cfg.layers[i])
        ids = {}
        for name in names:
            ids[name] = next_id[0]
            next_id[0] += 1
        return LayerCall(block=i, cache=ids[""] if names == [""] else ids)

    order = []
    if cfg.loop is None:
        order = [call(i) for i in range(n_layers)]
    else:
        lp = cfg.loop
        blocks.append(BlockSpec("reentry", None, None, None, None,
                                {"width": d, "passes": lp.times, "names": {"mix": "loop.in", "step": "loop.step"}}))
        order = [call(i) for i in range(lp.start)]
        for t in range(lp.times):
            order.append(LayerCall(block=n_layers, cache={}, arg=t))
            order += [call(i) for i in range(lp.start, lp.stop)]
        order += [call(i) for i in range(lp.stop, n_layers)]
    embedding, embedding_cache = None, None
    if cfg.bigram is not None:
        embedding = PartSpec("token_pair_table", dict(vocab_size=cfg.vocab, width=d, buckets=cfg.bigram.buckets,
                                                      mul_prev=cfg.bigram.mul_prev, mul_cur=cfg.bigram.mul_cur),
                             {"weight": "embed", "pairs": "bigram"})
        embedding_cache = next_id[0]
        next_id[0] += 1
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=d, blocks=blocks, order=order,
        final_norm=_tanh_norm(d, "final.norm"), embed_name="embed", embedding=embedding, embedding_cache=embedding_cache,
        keep_embedding=cfg.loop is not None,
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "width": d, "softcap": cfg.logit_softcap or 0.0}, {"weight": "head"}),
        eos_token_ids=cfg.eos_token_ids, max_position=cfg.max_position, strip_prefixes=())


register_architecture("Nolapel", NolapelConfig.from_dict, build_spec)
