"""A Tebalorn model as a list of parts.

Every layer is a ``parallel`` block with one norm: mixer and feed-forward both read norm1(x) and join
the stream together, then the per-layer token input (``gated_token_table``) is added where the model has
one.  Mixers: ``gla`` and ``lightning`` are ``linear_attention`` (a decay per key channel that the input
decides, a head norm and a silu gate; or silu on q, k and v, a constant decay per head, a norm over all
heads and a sigmoid gate); ``attention`` is ``wide_attention`` with sinks, YaRN-scaled rotation of a
head's leading part and a chunked mask.  Feed-forward: ``dense_glu`` with relu, or ``moe_topk_softmax``
with silu experts and a shared expert.  The embedding's rows are multiplied by ``embedding.scale``, the
logits by ``logit_scale``.  Tensor names: ``l<i>.norm1``, ``.mix.q|k|v|o``, ``.mix.g|norm`` and
``.mix.a1|a2|a2.b`` or ``.mix.sink``, ``.mlp.gate|up|down`` or ``.mlp.router|e<k>.*|shared.*``,
``.side.gate|proj|norm``; ``embed``, ``side.embed``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from .tebalorn import TebalornConfig
from .registry import register_architecture
from ..parts.base import PartSpec, BlockSpec, LayerCall, ModelSpec


def build_spec(cfg: TebalornConfig) -> ModelSpec:
    d, eps = cfg.width, cfg.norm_eps
    n_layers = len(cfg.layers)
    blocks, order = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        mx = layer.mixer
        names = {"q_proj": p + "mix.q", "k_proj": p + "mix.k", "v_proj": p + "mix.v", "o_proj": p + "mix.o"}
        if layer.type == "attention":
            position = None
            if mx.rot_base is not None and mx.rot_dims > 0:
                sc = mx.rot_scaling
                scaling = None if sc is None else {"rope_type": "yarn", "factor": sc.factor, "original": sc.original,
                                                   "fast": sc.fast, "slow": sc.slow}
                position = PartSpec("rotary", {"head_dim": mx.dim, "theta": mx.rot_base, "rotary_dim": mx.rot_dims,
                                               "scaling": scaling})
            names["sink"] = p + "mix.sink"
            mixer = PartSpec("wide_attention", dict(
                hidden_size=d, n_heads=mx.heads, n_kv_heads=mx.kv_heads, key_dim=mx.dim, value_dim=mx.vdim, scale=mx.scale,
                position=position, visibility="full" if mx.chunk is None else "chunk", span=mx.chunk or 0, norm_eps=eps,
                sinks=True), names)
        else:
            names.update({"gate_proj": p + "mix.g", "norm": p + "mix.norm"})
            args = dict(hidden_size=d, n_heads=mx.heads, key_dim=mx.dim, value_dim=mx.vdim, norm_eps=eps)
            if layer.type == "gla":
                names.update({"decay_down": p + "mix.a1", "decay_up": p + "mix.a2", "decay_bias": p + "mix.a2.b"})
                args.update(decay="channel", decay_tau=mx.tau, q_scale=float(mx.dim) ** -0.5, out_norm="head", gate="silu")
            else:
                args.update(decay="head", head_decay=list(mx.decay), activation="silu", out_norm="all", gate="sigmoid")
            mixer = PartSpec("linear_attention", args, names)
        ffn = None
        if layer.mlp is not None:
            f = p + "mlp."
            if layer.mlp.kind == "dense":
                ffn = PartSpec("dense_glu", dict(hidden_size=d, intermediate_size=layer.mlp.ff, activation="relu"),
                               {"gate_proj": f + "gate", "up_proj": f + "up", "down_proj": f + "down"})
            else:
                ml = layer.mlp
                fn = {"router": f + "router"}
                for e in range(ml.experts):
                    fn.update({f"e{e}.{k}": f"{f}e{e}.{k}" for k in ("gate", "up", "down")})
                if ml.shared_ff is not None:
                    fn.update({f"shared.{k}": f"{f}shared.{k}" for k in ("gate", "up", "down")})
                ffn = PartSpec("moe_topk_softmax", dict(
                    hidden_size=d, intermediate_size=ml.expert_ff, n_experts=ml.experts, top_k=ml.top,
                    shared_intermediate_size=ml.shared_ff, activation="silu"), fn)
        extra = {}
        if cfg.side_dim is not None:
            extra["side"] = PartSpec("gated_token_table", dict(
                vocab_size=cfg.vocab, width=d, dim=cfg.side_dim, n_layers=n_layers, layer=i, eps=eps, mult=1.0),
                {"embed": "side.embed", "gate": p + "side.gate", "proj": p + "side.proj", "norm": p + "side.norm"})
        norm1 = PartSpec("rms", {"width": d, "eps": eps}, {"weight": p + "norm1"})
        blocks.append(BlockSpec("parallel", norm1, mixer, None, ffn, extra))
        order.append(LayerCall(block=i, cache=i))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=d, blocks=blocks, order=order,
        final_norm=PartSpec("rms", {"width": d, "eps": eps}, {"weight": "final.norm"}),
        embedding=PartSpec("token_table", {"vocab_size": cfg.vocab, "width": d, "scale": cfg.embed_scale}, {"weight": "embed"}),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "width": d, "scale": cfg.logit_scale}, {"weight": "head"}),
        eos_token_ids=cfg.eos_token_ids, max_position=cfg.max_position, strip_prefixes=())


register_architecture("Tebalorn", TebalornConfig.from_dict, build_spec)
