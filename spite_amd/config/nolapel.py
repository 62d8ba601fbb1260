"""Typed configuration of the Nolapel design, read from the keys of its ``config.json``.

``architecture`` names the design; ``vocab``, ``width``, ``norm.eps``, ``logit_softcap`` and ``embedding.bigram``
(``buckets``, ``mul_prev``, ``mul_cur``: a second embedding chosen by a hash of the token and the one before) are
the model's own; ``layers`` lists the layers in order, each with its ``type`` (the kind of mixer), the mixer's sizes
and constants under ``mixer`` and its feed-forward under ``mlp`` (``null``: none); ``loop`` (``start``, ``stop``,
``times``) names a run of layers that is walked several times with the same weights.  Three kinds of mixer:

* ``attention``: grouped-query attention whose values are its keys, with a short convolution on q and k (``conv``
  taps), a norm per head, a query temperature (``q_temp``: ``coef``, ``every``), per-head slopes on the distance, a
  sliding window (``mask.size``), a sink of score zero and ``scale`` on the scores;
* ``parallel``: two mixers side by side, ``left`` (attention with a rotation of a head's leading part, ``rot``:
  ``base``, ``dims``; a learned sink a head; every earlier key) and ``right`` (time mixing with a decayed state per
  head: ``heads``, ``dim``), added with ``left_scale`` and ``right_scale``;
* ``mamba2``: a state-space mixer (``heads``, ``vdim``, ``state``, ``groups``, ``conv`` taps, ``norm_groups``).

The feed-forward is a mixture of experts (``router.experts``, ``router.top``, ``expert.ff``, ``shared.ff``).
Every size and constant is read here; every problem found is reported in one ``ConfigError``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .llama4 import ConfigError

MIXER_TYPES = ("attention", "parallel", "mamba2")


@dataclass(frozen=True)
class NolapelAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int] = None          # mask.size; None: every earlier key
    conv: int = 0                         # taps of the convolution on q and k (0: none)
    q_temp: Optional[Tuple[float, int]] = None   # (coef, every)
    rot_base: Optional[float] = None      # the rotated kind (left half of ``parallel``)
    rot_dims: int = 0


@dataclass(frozen=True)
class NolapelTimeMix:
    heads: int
    dim: int


@dataclass(frozen=True)
class NolapelStateSpace:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int


@dataclass(frozen=True)
class NolapelMlp:
    experts: int
    top: int
    expert_ff: int
    shared_ff: Optional[int]


@dataclass(frozen=True)
class NolapelLayer:
    type: str
    mixer: Any                            # NolapelAttention | (NolapelAttention, NolapelTimeMix, left_scale, right_scale) | NolapelStateSpace
    mlp: Optional[NolapelMlp]


@dataclass(frozen=True)
class NolapelLoop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class NolapelBigram:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class NolapelConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    logit_softcap: Optional[float]
    bigram: Optional[NolapelBigram]
    loop: Optional[NolapelLoop]
    layers: Tuple[NolapelLayer, ...]
    torch_dtype: str = "bfloat16"
    eos_token_ids: Tuple[int, ...] = ()
    max_position: int = 1 << 20

    @staticmethod
    def from_dict(raw: Mapping[str, Any]) -> "NolapelConfig":
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

        def attention(mx, w, rotated):
            mask, qt, rot = mx.get("mask"), mx.get("q_temp"), mx.get("rot")
            a = NolapelAttention(
                heads=need(mx, "heads", int, w), kv_heads=need(mx, "kv_heads", int, w), dim=need(mx, "dim", int, w),
                vdim=need(mx, "vdim", int, w), scale=need(mx, "scale", float, w),
                window=None if mask is None else need(mask, "size", int, w + "mask."),
                conv=0 if mx.get("conv") is None else need(mx, "conv", int, w),
                q_temp=None if qt is None else (need(qt, "coef", float, w + "q_temp.", positive=False), need(qt, "every", int, w + "q_temp.")),
                rot_base=None if rot is None else need(rot, "base", float, w + "rot."),
                rot_dims=0 if rot is None else need(rot, "dims", int, w + "rot."))
            if a.heads % a.kv_heads:
                problems.append(f"{w}heads = {a.heads} is no multiple of kv_heads = {a.kv_heads}")
            if a.rot_dims % 2 or a.rot_dims > a.dim:
                problems.append(f"{w}rot.dims = {a.rot_dims} must be even and at most dim = {a.dim}")
            if not rotated and a.vdim != a.dim:
                problems.append(f"{w}vdim = {a.vdim}: the values are the keys, so it must equal dim = {a.dim}")
            return a

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
            if kind == "attention":
                mixer = attention(mx, wm, rotated=False)
            elif kind == "parallel":
                left, right = mx.get("left") or {}, mx.get("right") or {}
                mixer = (attention(left, wm + "left.", rotated=True),
                         NolapelTimeMix(heads=need(right, "heads", int, wm + "right."), dim=need(right, "dim", int, wm + "right.")),
                         need(mx, "left_scale", float, wm, positive=False), need(mx, "right_scale", float, wm, positive=False))
            else:
                mixer = NolapelStateSpace(heads=need(mx, "heads", int, wm), vdim=need(mx, "vdim", int, wm),
                                          state=need(mx, "state", int, wm), groups=need(mx, "groups", int, wm),
                                          conv=need(mx, "conv", int, wm), norm_groups=need(mx, "norm_groups", int, wm))
                if mixer.heads % mixer.groups:
                    problems.append(f"{wm}heads = {mixer.heads} is no multiple of groups = {mixer.groups}")
                if (mixer.heads * mixer.vdim) % mixer.norm_groups:
                    problems.append(f"{wm}norm_groups = {mixer.norm_groups} does not divide heads * vdim")
            mlp = None
            rm = L.get("mlp")
            if rm is not None:
                wl = w + "mlp."
                if rm.get("kind", "moe") != "moe":
                    problems.append(f"{wl}kind = {rm.get('kind')!r} (known: moe)")
                router, shared = rm.get("router") or {}, rm.get("shared")
                mlp = NolapelMlp(experts=need(router, "experts", int, wl + "router."), top=need(router, "top", int, wl + "router."),
                                 expert_ff=need(rm.get("expert") or {}, "ff", int, wl + "expert."),
                                 shared_ff=None if shared is None else need(shared, "ff", int, wl + "shared."))
                if mlp.top > mlp.experts:
                    problems.append(f"{wl}router.top = {mlp.top} of {mlp.experts} experts")
            layers.append(NolapelLayer(kind, mixer, mlp))
        loop = None
        rl = raw.get("loop")
        if rl is not None:
            loop = NolapelLoop(start=need(rl, "start", int, "loop.", positive=False), stop=need(rl, "stop", int, "loop."),
                               times=need(rl, "times", int, "loop."))
            if not 0 <= loop.start < loop.stop <= max(len(raw_layers), 1):
                problems.append(f"loop: layers {loop.start} .. {loop.stop - 1} of {len(raw_layers)}")
        bg = (raw.get("embedding") or {}).get("bigram")
        bigram = None if bg is None else NolapelBigram(
            buckets=need(bg, "buckets", int, "embedding.bigram."), mul_prev=need(bg, "mul_prev", int, "embedding.bigram.", positive=False),
            mul_cur=need(bg, "mul_cur", int, "embedding.bigram.", positive=False))
        cfg = NolapelConfig(
            architecture=str(raw.get("architecture", "Nolapel")),
            vocab=need(raw, "vocab", int, ""), width=need(raw, "width", int, ""),
            norm_eps=need(raw.get("norm") or {}, "eps", float, "norm."),
            logit_softcap=None if raw.get("logit_softcap") is None else need(raw, "logit_softcap", float, ""),
            bigram=bigram, loop=loop, layers=tuple(layers), torch_dtype=str(raw.get("torch_dtype", "bfloat16")),
            eos_token_ids=tuple(int(t) for t in raw.get("eos_token_ids", ()) or ()),
            max_position=int(raw.get("max_position", 1 << 20)))
        if problems:
            raise ConfigError("config.json does not describe a Nolapel model: " + "; ".join(problems))
        return cfg
