"""Typed configuration of the Tebalorn design, read from the keys of its ``config.json``.

``architecture`` names the design; ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``,
``logit_scale`` and ``token_side.dim`` are the model's own; ``layers`` lists the layers in order,
each with its ``type`` (the kind of mixer), the mixer's sizes and constants under ``mixer`` and
its feed-forward under ``mlp`` (``null``: none).  Three kinds of mixer:

* ``gla``: linear attention with a state per head and a decay per key channel that the input
  decides (``heads``, ``dim``, ``vdim``, ``tau``; the decay's inner width is the shape of its first matrix);
* ``lightning``: linear attention with one constant decay per head (``heads``, ``dim``, ``vdim``, ``decay``);
* ``attention``: grouped-query softmax attention with a sink per head, keys and values of their own
  widths, a rotation of a head's leading part with YaRN-scaled frequencies (``rot``: ``base``,
  ``dims``, ``scaling``: ``factor``, ``original``, ``fast``, ``slow``), a chunked or full mask
  (``mask.size``) and ``scale`` on the scores.

Every size and constant is read here; every problem found is reported in one ``ConfigError``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .llama4 import ConfigError

MIXER_TYPES = ("gla", "lightning", "attention")
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class YarnScaling:
    factor: float
    original: float               # the context length that the frequencies were trained at
    fast: float                   # rotations within ``original`` above which a frequency is kept
    slow: float                   # ... below which it is divided by ``factor``


@dataclass(frozen=True)
class TebalornMixer:
    heads: int
    dim: int                      # query/key size of a head
    vdim: int                     # value size of a head
    # gla
    tau: float = 1.0
    # lightning
    decay: Tuple[float, ...] = ()
    # attention
    kv_heads: int = 0
    scale: float = 1.0
    chunk: Optional[int] = None   # mask.size; None: every earlier key
    rot_base: Optional[float] = None
    rot_dims: int = 0
    rot_scaling: Optional[YarnScaling] = None


@dataclass(frozen=True)
class TebalornMlp:
    kind: str                     # "dense" | "moe"
    ff: int = 0                   # dense: inner width
    experts: int = 0
    top: int = 0
    expert_ff: int = 0
    shared_ff: Optional[int] = None


@dataclass(frozen=True)
class TebalornLayer:
    type: str
    mixer: TebalornMixer
    mlp: Optional[TebalornMlp]


@dataclass(frozen=True)
class TebalornConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    embed_scale: float
    logit_scale: float
    side_dim: Optional[int]       # token_side.dim; None: no per-layer token input
    layers: Tuple[TebalornLayer, ...]
    torch_dtype: str = "bfloat16"
    eos_token_ids: Tuple[int, ...] = ()
    max_position: int = 1 << 20

    @staticmethod
    def from_dict(raw: Mapping[str, Any]) -> "TebalornConfig":
        problems = []

        def need(d, key, kind, where, positive=True):
            if not isinstance(d, Mapping) or key not in d or d[key] is None:
                problems.append(f"{where}{key} is missing")
                return kind(1)
            try:
                v = kind(d[key])
            except (TypeError, ValueError):
                problems.append(f"{where}{key} = {d[key]!r} is no {kind.__name__}")
                return kind(1)
            if positive and not v > 0:
                problems.append(f"{where}{key} = {v} must be positive")
            return v

        layers = []
        raw_layers = raw.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            problems.append("layers is missing or empty")
            raw_layers = []
        for i, L in enumerate(raw_layers):
            w = f"layers[{i}]."
            kind = L.get("type") if isinstance(L, Mapping) else None
            if kind not in MIXER_TYPES:
                problems.append(f"{w}type = {kind!r} (known: {', '.join(MIXER_TYPES)})")
                continue
            mx = L.get("mixer") or {}
            wm = w + "mixer."
            common = dict(heads=need(mx, "heads", int, wm), dim=need(mx, "dim", int, wm), vdim=need(mx, "vdim", int, wm))
            if kind == "gla":
                mixer = TebalornMixer(**common, tau=need(mx, "tau", float, wm))
            elif kind == "lightning":
                decay = mx.get("decay")
                if not isinstance(decay, (list, tuple)) or len(decay) != common["heads"]:
                    problems.append(f"{wm}decay must list one number for each of the {common['heads']} heads")
                    decay = [1.0] * common["heads"]
                try:
                    decay = tuple(float(x) for x in decay)
                except (TypeError, ValueError):
                    problems.append(f"{wm}decay holds something that is no number")
                    decay = (1.0,) * common["heads"]
                if any(not 0.0 <= x <= 1.0 for x in decay):
                    problems.append(f"{wm}decay must lie in [0, 1]")
                mixer = TebalornMixer(**common, decay=decay)
            else:
                mask, rot = mx.get("mask"), mx.get("rot")
                chunk = None if mask is None else need(mask, "size", int, wm + "mask.")
                rot_base, rot_dims, scaling = None, 0, None
                if rot is not None:
                    rot_base, rot_dims = need(rot, "base", float, wm + "rot."), need(rot, "dims", int, wm + "rot.")
                    sc = rot.get("scaling")
                    if sc is not None:
                        ws = wm + "rot.scaling."
                        scaling = YarnScaling(factor=need(sc, "factor", float, ws), original=need(sc, "original", float, ws),
                                              fast=need(sc, "fast", float, ws), slow=need(sc, "slow", float, ws))
                mixer = TebalornMixer(**common, kv_heads=need(mx, "kv_heads", int, wm), scale=need(mx, "scale", float, wm),
                                      chunk=chunk, rot_base=rot_base, rot_dims=rot_dims, rot_scaling=scaling)
                if mixer.heads % mixer.kv_heads:
                    problems.append(f"{wm}heads = {mixer.heads} is no multiple of kv_heads = {mixer.kv_heads}")
                if mixer.rot_dims % 2 or mixer.rot_dims > mixer.dim:
                    problems.append(f"{wm}rot.dims = {mixer.rot_dims} must be even and at most dim = {mixer.dim}")
            mlp = None
            rm = L.get("mlp")
            if rm is not None:
                wl = w + "mlp."
                k = rm.get("kind") if isinstance(rm, Mapping) else None
                if k == "dense":
                    mlp = TebalornMlp("dense", ff=need(rm, "ff", int, wl))
                elif k == "moe":
                    router, shared = rm.get("router") or {}, rm.get("shared")
                    mlp = TebalornMlp("moe", experts=need(router, "experts", int, wl + "router."),
                                      top=need(router, "top", int, wl + "router."),
                                      expert_ff=need(rm.get("expert") or {}, "ff", int, wl + "expert."),
                                      shared_ff=None if shared is None else need(shared, "ff", int, wl + "shared."))
                    if mlp.top > mlp.experts:
                        problems.append(f"{wl}router.top = {mlp.top} of {mlp.experts} experts")
                else:
                    problems.append(f"{wl}kind = {k!r} (known: {', '.join(MLP_KINDS)})")
            layers.append(TebalornLayer(kind, mixer, mlp))
        emb, side = raw.get("embedding"), raw.get("token_side")
        cfg = TebalornConfig(
            architecture=str(raw.get("architecture", "Tebalorn")),
            vocab=need(raw, "vocab", int, ""), width=need(raw, "width", int, ""),
            norm_eps=need(raw.get("norm") or {}, "eps", float, "norm."),
            embed_scale=1.0 if emb is None else need(emb, "scale", float, "embedding.", positive=False),
            logit_scale=1.0 if raw.get("logit_scale") is None else need(raw, "logit_scale", float, "", positive=False),
            side_dim=None if side is None else need(side, "dim", int, "token_side."),
            layers=tuple(layers), torch_dtype=str(raw.get("torch_dtype", "bfloat16")),
            eos_token_ids=tuple(int(t) for t in raw.get("eos_token_ids", ()) or ()),
            max_position=int(raw.get("max_position", 1 << 20)))
        if problems:
            raise ConfigError("config.json does not describe a Tebalorn model: " + "; ".join(problems))
        return cfg
