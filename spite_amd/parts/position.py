"""Position encodings of the attention mixer.

``rotary``: rotation by pos * f_i on pairs of every query and key head
(crates/spite-rope/src/lib.rs:78-92; half-split pairs (i, i+hd/2) as there, or adjacent
pairs), f_i = theta^(-2i/hd), optionally rescaled once at load by the ``llama3`` rule
(wavelength L = 2*pi/f: L < orig/high keeps f; L > orig/low gives f/factor; between, the
blend (1-s)*f/factor + s*f with s = (orig/L - low)/(high - low)) or by the ``linear`` rule
(every f divided by ``factor``: positions counted in units of ``factor`` tokens) or by the ``yarn`` rule:
with n(t) = rot * ln(orig / (2 pi t)) / (2 ln theta), the index of the pair that turns t times within
``orig`` positions, lo = max(floor(n(fast)), 0), hi = min(ceil(n(slow)), rot - 1) and the ramp
r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), the frequency becomes (1 - r_i) f_i + r_i f_i / factor:
pairs that turn often keep theirs, slow pairs are stretched; sine and cosine are then both multiplied by
the ``magnitude`` 0.1 ln(factor) + 1 (a mixer whose kernel knows no magnitude refuses the encoding).  The
table is computed in float64 and stored as fp32; angle and rotation are fp32 in the kernel.

``distance_slopes``: nothing is done to q and k; head h's score of (query at i, key at j) loses
slope_h * (i - j) with slope_h = 2^(-ratio (h + 1) / H), H the number of heads: the further a key, the less it counts,
each head at its own rate.

``none``: no position information (NoPE layers).
"""
from __future__ import annotations

import math

import torch

from .base import PositionEncoding, register


def rotation_magnitude(scaling=None) -> float:
    """What sine and cosine are multiplied by (1 unless the scaling rule brings a constant)."""
    if scaling is not None and scaling.get("rope_type", "llama3") == "yarn":
        return 0.1 * math.log(float(scaling["factor"])) + 1.0
    return 1.0


def inv_frequencies(head_dim: int, theta: float, scaling=None):
    half = head_dim // 2
    out = []
    yarn = None
    if scaling is not None and scaling.get("rope_type", "llama3") == "yarn":
        factor, orig = float(scaling["factor"]), float(scaling["original"])
        index_of = lambda turns: head_dim * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(theta)))
        lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(index_of(float(scaling["slow"]))), head_dim - 1)
        yarn = (factor, lo, hi)
    for i in range(half):
        f = 1.0 / (float(theta) ** (2.0 * i / head_dim))
        if yarn is not None:
            factor, lo, hi = yarn
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f = f / factor * ramp + f * (1.0 - ramp)
        elif scaling is not None and scaling.get("rope_type", "llama3") == "linear":
            f = f / float(scaling["factor"])
        elif scaling is not None:
            factor, low, high, orig = (float(scaling["factor"]), float(scaling["low_freq_factor"]),
                                       float(scaling["high_freq_factor"]),
                                       float(scaling["original_max_position_embeddings"]))
            wavelen = 2.0 * math.pi / f
            if wavelen < orig / high:
                pass
            elif wavelen > orig / low:
                f = f / factor
            else:
                s = (orig / wavelen - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


@register("position", "rotary")
class Rotary(PositionEncoding):
    graph_safe = True

    def __init__(self, env, head_dim: int, theta: float, scaling=None, pairing: str = "half", rotary_dim=None):
        """``rotary_dim``: only the first so many elements of a head rotate, with the frequencies of
        a head of that size; the rest pass through (default: the whole head)."""
        rot = head_dim if rotary_dim is None else int(rotary_dim)
        if head_dim % 2 or rot % 2 or not 0 < rot <= head_dim:
            raise ValueError(f"rotary: head size {head_dim} and rotating part {rot} must be even, the part within the head")
        if pairing not in ("half", "adjacent"):
            raise ValueError(f"rotary: pairing {pairing!r}")
        if scaling is not None and scaling.get("rope_type", "llama3") not in ("llama3", "linear", "yarn"):
            raise ValueError(f"rotary: scaling of type {scaling.get('rope_type')!r} is not known")
        self.adjacent = pairing == "adjacent"
        self.rotary_dim = rot
        self.magnitude = rotation_magnitude(scaling)
        self.inv_freq = torch.tensor(inv_frequencies(rot, theta, scaling), dtype=torch.float64) \
            .to(torch.float32).to(env.device)

    def kernel_args(self):
        return {"use_rope": True, "inv_freq": self.inv_freq, "adjacent": self.adjacent, "rotary_dim": self.rotary_dim,
                "magnitude": self.magnitude}


@register("position", "none")
class NoPosition(PositionEncoding):
    graph_safe = True

    def __init__(self, env):
        pass


@register("position", "distance_slopes")
class DistanceSlopes(PositionEncoding):
    graph_safe = True

    def __init__(self, env, ratio: float = 8.0):
        self.env, self.ratio = env, float(ratio)

    def score_slopes(self, n_heads: int):
        vals = [2.0 ** (-self.ratio * (h + 1) / n_heads) for h in range(n_heads)]
        return torch.tensor(vals, dtype=torch.float64).to(torch.float32).to(self.env.device)
