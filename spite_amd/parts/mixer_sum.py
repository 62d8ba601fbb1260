"""Several mixers side by side: all read the same input and their results are added, each times a constant.

``mixer_sum(parts={name: PartSpec}, scales={name: constant})``.  The tensors and the caches of a part carry its name
before their own (``left.q_proj``; cache ``left`` or, for a part with several caches, ``right.state``).
"""
from __future__ import annotations

import torch

from .base import Mixer, register, build as build_part
from ..csrc import hipops


@register("mixer", "mixer_sum")
class MixerSum(Mixer):
    def __init__(self, env, parts, scales=None):
        if not parts:
            raise ValueError("mixer_sum: no parts")
        self.env = env
        self.names = list(parts)
        self.parts = {name: build_part("mixer", spec, env) for name, spec in parts.items()}
        self.scales = {name: float((scales or {}).get(name, 1.0)) for name in self.names}
        self.graph_safe = all(p.graph_safe for p in self.parts.values())
        self.step_arrays = tuple(sorted({a for p in self.parts.values() for a in p.step_arrays}))

    def params(self):
        return {f"{name}.{local}": ps for name, part in self.parts.items() for local, ps in part.params().items()}

    def load(self, tensors):
        for name, part in self.parts.items():
            pre = name + "."
            part.load({k[len(pre):]: v for k, v in tensors.items() if k.startswith(pre)})

    def slow_paths(self, page_size):
        return [f"{name}: {note}" for name, part in self.parts.items() for note in part.slow_paths(page_size)]

    def cache_needs(self):
        needs = {}
        for name, part in self.parts.items():
            for local, need in part.cache_needs().items():
                needs[name if local == "" else f"{name}.{local}"] = need
        return needs

    def _cache_of(self, name, part, cache):
        locals_ = list(part.cache_needs())
        if locals_ == [""]:
            return cache[name]
        return {local: cache[f"{name}.{local}"] for local in locals_}

    def forward(self, x, ctx, cache):
        outs = [(self.scales[name], part.forward(x, ctx, self._cache_of(name, part, cache))) for name, part in self.parts.items()]
        a, total = outs[0]
        if len(outs) == 1:
            if a != 1.0:
                hipops.scale_rows(total, a)
            return total
        for i, (b, y) in enumerate(outs[1:]):
            hipops.axpby_rows(total, y, total, a if i == 0 else 1.0, b)
        return total
