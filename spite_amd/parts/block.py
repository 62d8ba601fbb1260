"""Arrangements of a layer.  ``prenorm``: pre-norm residual block,
h += mixer(norm1(h)); h += ffn(norm2(h)) (crates/spite-models/src/llama/llama4.rs:126-127,
202-211, 272-274).  The additions are folded into the norm that follows them: a block hands
its last increments to the next block (or the final norm) instead of adding them itself."""
from __future__ import annotations

import torch

from .base import Block, NormedIncrement, NORMED_INCREMENTS, register, build as build_part, two_increments


@register("block", "prenorm")
class PreNormBlock(Block):
    graph_safe = True

    def __init__(self, env, spec):
        self.env = env
        self.norm1 = build_part("norm", spec.norm1, env)
        self.mixer = build_part("mixer", spec.mixer, env)
        self.norm2 = build_part("norm", spec.norm2, env)
        self.ffn = build_part("ffn", spec.ffn, env)
        self.children = (("norm1", self.norm1, spec.norm1), ("mixer", self.mixer, spec.mixer),
                         ("norm2", self.norm2, spec.norm2), ("ffn", self.ffn, spec.ffn))
        self.graph_safe = all(part.graph_safe for _, part, _ in self.children)
        self.step_arrays = tuple(sorted({a for _, part, _ in self.children for a in part.step_arrays}))

    def forward(self, h, pending, ctx, cache):
        state = {"h": h, "pending": pending}
        for _, stage in self.stages():
            stage(state, ctx, cache)
        return state["pending"]

    def stages(self):
        # first norm | mixer | second norm and feed-forward: a mixer that reads the step's metadata
        # on the host keeps only itself out of a graph
        return [(self.norm1.graph_safe, self._stage_norm1), (self.mixer.graph_safe, self._stage_mixer),
                (self.norm2.graph_safe and self.ffn.graph_safe, self._stage_ffn)]

    def _stage_norm1(self, state, ctx, cache):
        h = state["h"]
        d1, d2 = two_increments(h, state["pending"])
        n = ctx.ws.take(tuple(h.shape), self.env.dtype)
        self.norm1.forward(h, n, d1=d1, d2=d2)
        state["normed"] = n

    def _stage_mixer(self, state, ctx, cache):
        state["mixed"] = self.mixer.forward(state.pop("normed"), ctx, cache)

    def _stage_ffn(self, state, ctx, cache):
        h, delta, ws = state["h"], state.pop("mixed"), ctx.ws
        T, d = h.shape
        n2 = ws.take((T, d), self.env.dtype)
        proj = self.ffn.input_projection()
        if proj is not None and self.norm2.can_project(proj):
            # the norm forms the feed-forward's small fp32 products (router logits) itself
            logits = ws.take((T, proj.shape[0]), torch.float32)
            self.norm2.forward(h, n2, d1=delta, proj=proj, proj_out=logits)
            state["pending"] = tuple(self.ffn.forward(n2, None, ctx, projected=logits))
            return
        n2_32 = None
        if self.ffn.wants_f32_input:
            n2_32 = n2 if n2.dtype == torch.float32 else ws.take((T, d), torch.float32)
        self.norm2.forward(h, n2, d1=delta, out32=None if n2_32 is n2 else n2_32)
        state["pending"] = tuple(self.ffn.forward(n2, n2_32, ctx))


@register("block", "sandwich")
class SandwichBlock(Block):
    """Every sublayer has a norm before it and one after it, and its normed result joins the
    stream times a constant m:  h += m * norm1b(mixer(norm1(h)));  h += m * norm2b(ffn(norm2(h)));
    then, if the layer has one, a side input from the step's tokens (``spec.extra["side"]``).  The
    feed-forward may be missing.  ``spec.extra``: ``norm1b``, ``norm2b`` (PartSpecs), ``residual_mult``.
    Every addition is folded into the norm kernel that next reads the stream (a normed increment
    beside the plain ones); the last one is handed to the next block.  The norms are of any kind that
    offers ``as_increment`` (RMS, tanh).  A mixer with several caches (``Mixer.cache_needs``) gets them by name."""
    graph_safe = True

    def __init__(self, env, spec):
        self.env = env
        ex = spec.extra
        self.mult = float(ex.get("residual_mult", 1.0))
        self.norm1 = build_part("norm", spec.norm1, env)
        self.mixer = build_part("mixer", spec.mixer, env)
        self.norm1b = build_part("norm", ex["norm1b"], env)
        self.children = [("norm1", self.norm1, spec.norm1), ("mixer", self.mixer, spec.mixer),
                         ("norm1b", self.norm1b, ex["norm1b"])]
        self.norm2 = self.ffn = self.norm2b = self.side = None
        if spec.ffn is not None:
            self.norm2 = build_part("norm", spec.norm2, env)
            self.ffn = build_part("ffn", spec.ffn, env)
            self.norm2b = build_part("norm", ex["norm2b"], env)
            self.children += [("norm2", self.norm2, spec.norm2), ("ffn", self.ffn, spec.ffn),
                              ("norm2b", self.norm2b, ex["norm2b"])]
        if ex.get("side") is not None:
            self.side = build_part("side", ex["side"], env)
            self.children.append(("side", self.side, ex["side"]))
        self.children = tuple(self.children)
        self.graph_safe = all(part.graph_safe for _, part, _ in self.children)
        self.step_arrays = tuple(sorted({a for _, part, _ in self.children for a in part.step_arrays}))

    def cache_needs(self):
        return self.mixer.cache_needs()

    def forward(self, h, pending, ctx, cache):
        state = {"h": h, "pending": pending}
        for _, stage in self.stages():
            stage(state, ctx, cache)
        return state["pending"]

    def stages(self):
        rest = all(p.graph_safe for p in (self.norm2, self.ffn, self.side) if p is not None)
        return [(self.norm1.graph_safe, self._stage_norm1), (self.mixer.graph_safe, self._stage_mixer),
                (rest, self._stage_rest)]

    @staticmethod
    def _split(h, pending, norm=None):
        """(d1, d2, one normed increment or None) of what is still to be added to h; the normed increment is one
        that ``norm`` (default: an RMS norm) adds in its own pass."""
        takes = norm.takes if norm is not None and hasattr(norm, "takes") else (lambda p: isinstance(p, NormedIncrement))
        normed = [p for p in pending if isinstance(p, NORMED_INCREMENTS) and takes(p)]
        last = normed.pop() if normed else None
        d1, d2 = two_increments(h, tuple(p for p in pending if p is not last))
        return d1, d2, (last.as_arg() if last is not None else None)

    def _stage_norm1(self, state, ctx, cache):
        h = state["h"]
        d1, d2, normed = self._split(h, state["pending"], self.norm1)
        n = ctx.ws.take(tuple(h.shape), self.env.dtype)
        self.norm1.forward(h, n, d1=d1, d2=d2, normed=normed)
        state["normed"] = n

    def _stage_mixer(self, state, ctx, cache):
        state["mixed"] = self.mixer.forward(state.pop("normed"), ctx, cache)

    def _stage_rest(self, state, ctx, cache):
        h, ws = state["h"], ctx.ws
        T, d = h.shape
        pend = (self.norm1b.as_increment(state.pop("mixed"), self.mult),)
        if self.ffn is not None:
            n2 = ws.take((T, d), self.env.dtype)
            proj = self.ffn.input_projection()
            if proj is not None and self.norm2.can_project(proj):
                logits = ws.take((T, proj.shape[0]), torch.float32)
                self.norm2.forward(h, n2, normed=pend[0].as_arg(), proj=proj, proj_out=logits)
                f = tuple(self.ffn.forward(n2, None, ctx, projected=logits))
            else:
                n2_32 = None
                if self.ffn.wants_f32_input:
                    n2_32 = n2 if n2.dtype == torch.float32 else ws.take((T, d), torch.float32)
                self.norm2.forward(h, n2, normed=pend[0].as_arg(), out32=None if n2_32 is n2 else n2_32)
                f = tuple(self.ffn.forward(n2, n2_32, ctx))
            from ..csrc import hipops
            for extra in f[1:]:                      # a feed-forward with several results: the norm wants their sum
                hipops.add_into(f[0], extra[:T])
            pend = (self.norm2b.as_increment(f[0], self.mult),)
        if self.side is not None:
            pend = tuple(self.side.forward(h, pend, ctx))
        state["pending"] = pend


@register("block", "parallel")
class ParallelBlock(Block):
    """Mixer and feed-forward read the same stream and their results join it together:
    h += mixer(shift(norm1(h))) + ffn(norm2(h)), each through a norm of its own, or, where the spec
    names no second norm, both through the one norm: h += mixer(n) + ffn(n), n = norm1(h).
    ``spec.extra["shift"]`` (a PartSpec of category ``shift``, optional) stands between the first norm
    and the mixer and keeps a state row per request; the feed-forward may be missing;
    ``spec.extra["side"]`` (category ``side``, optional) adds its input from the step's tokens to the
    stream after both.  The results are handed to the next block, whose first norm adds them."""
    graph_safe = True

    def __init__(self, env, spec):
        self.env = env
        self.norm1 = build_part("norm", spec.norm1, env)
        self.mixer = build_part("mixer", spec.mixer, env)
        self.children = [("norm1", self.norm1, spec.norm1), ("mixer", self.mixer, spec.mixer)]
        self.shift = self.norm2 = self.ffn = self.side = None
        sh = spec.extra.get("shift")
        if sh is not None:
            self.shift = build_part("shift", sh, env)
            self.children.append(("shift", self.shift, sh))
        if spec.ffn is not None:
            if spec.norm2 is not None:
                self.norm2 = build_part("norm", spec.norm2, env)
                self.children.append(("norm2", self.norm2, spec.norm2))
            self.ffn = build_part("ffn", spec.ffn, env)
            self.children.append(("ffn", self.ffn, spec.ffn))
        if spec.extra.get("side") is not None:
            self.side = build_part("side", spec.extra["side"], env)
            self.children.append(("side", self.side, spec.extra["side"]))
        self.children = tuple(self.children)
        self.graph_safe = all(part.graph_safe for _, part, _ in self.children)
        self.step_arrays = tuple(sorted({a for _, part, _ in self.children for a in part.step_arrays}))

    def cache_needs(self):
        needs = {"mixer": self.mixer.cache_need()}
        if self.shift is not None and self.shift.state_need() is not None:
            from .base import CacheNeed
            needs["shift"] = CacheNeed(state=self.shift.state_need())
        return needs

    def forward(self, h, pending, ctx, cache):
        state = {"h": h, "pending": pending}
        for _, stage in self.stages():
            stage(state, ctx, cache)
        return state["pending"]

    def stages(self):
        first = all(p.graph_safe for p in (self.norm1, self.shift, self.norm2) if p is not None)
        last = all(p.graph_safe for p in (self.ffn, self.side) if p is not None)
        return [(first, self._stage_norms), (self.mixer.graph_safe, self._stage_mixer), (last, self._stage_ffn)]

    def _stage_norms(self, state, ctx, cache):
        h, ws = state["h"], ctx.ws
        T, d = h.shape
        d1, d2, normed = SandwichBlock._split(h, state["pending"])
        extra = {} if normed is None else {"normed": normed}
        if self.ffn is not None and self.norm2 is None:
            self._one_norm(state, ctx, cache, d1, d2, extra)
            return
        n2 = n2_32 = None
        if self.ffn is not None:
            n2 = ws.take((T, d), self.env.dtype)
            if self.ffn.wants_f32_input:
                n2_32 = n2 if n2.dtype == torch.float32 else ws.take((T, d), torch.float32)
        # both norms of the stream in one pass where the first norm's kernel can do that
        paired = n2 is not None and n2_32 is None and getattr(self.norm1, "pairs_with", lambda o: False)(self.norm2)
        both = {"second": (self.norm2, n2)} if paired else {}
        if self.shift is not None:
            # the shift blends fp32 rows; the mixer's input takes the run's dtype after it
            n32 = ws.take((T, d), torch.float32)
            self.norm1.forward(h, None, d1=d1, d2=d2, out32=n32, **both, **extra)
            x = ws.take((T, d), self.env.dtype)
            self.shift.forward(n32, x, ctx, cache["shift"].state)        # a block with a shift has two caches, by name
        else:
            x = ws.take((T, d), self.env.dtype)
            self.norm1.forward(h, x, d1=d1, d2=d2, **both, **extra)
        state["mixer_in"] = x
        if self.ffn is not None:
            if not paired:
                # the same stream (the increments are in it now) through the second norm
                self.norm2.forward(h, n2, out32=None if n2_32 is n2 else n2_32, write_h=False)
            state["ffn_in"] = (n2, n2_32, None)

    def _one_norm(self, state, ctx, cache, d1, d2, extra):
        """One norm for both sublayers: its rows are the feed-forward's input and (through the shift, if
        there is one) the mixer's; the feed-forward's small fp32 products (router logits) are formed in the
        same pass where the norm can do that."""
        h, ws = state["h"], ctx.ws
        T, d = h.shape
        n = ws.take((T, d), self.env.dtype)
        proj = self.ffn.input_projection()
        n32 = logits = None
        if self.shift is not None or (self.ffn.wants_f32_input and not (proj is not None and self.norm1.can_project(proj))):
            n32 = n if n.dtype == torch.float32 and self.shift is None else ws.take((T, d), torch.float32)
        if proj is not None and self.norm1.can_project(proj):
            logits = ws.take((T, proj.shape[0]), torch.float32)
            self.norm1.forward(h, n, d1=d1, d2=d2, out32=None if n32 is n else n32, proj=proj, proj_out=logits, **extra)
        else:
            self.norm1.forward(h, n, d1=d1, d2=d2, out32=None if n32 is n else n32, **extra)
        x = n
        if self.shift is not None:
            x = ws.take((T, d), self.env.dtype)
            self.shift.forward(n32, x, ctx, cache["shift"].state)
        state["mixer_in"] = x
        state["ffn_in"] = (n, n32 if self.ffn.wants_f32_input and logits is None else None, logits)

    def _stage_mixer(self, state, ctx, cache):
        state["mixed"] = self.mixer.forward(state.pop("mixer_in"), ctx, cache["mixer"] if isinstance(cache, dict) else cache)

    def _stage_ffn(self, state, ctx, cache):
        pend = (state.pop("mixed"),)
        if self.ffn is not None:
            n2, n2_32, logits = state.pop("ffn_in")
            if logits is not None:
                pend += tuple(self.ffn.forward(n2, None, ctx, projected=logits))
            else:
                pend += tuple(self.ffn.forward(n2, n2_32, ctx))
        if self.side is not None:
            pend = tuple(self.side.forward(state["h"], pend, ctx))
        state["pending"] = pend


@register("block", "reentry")
class ReentryBlock(Block):
    """No layer, but what stands before a run of layers that is walked several times with the same weights: the
    stream is mixed with the embedding's result again and a vector of the pass is added,

        x <- W [x ; x0] + step[pass],

    W ``[d, 2d]`` (the stream's columns first), x0 what the embedding left at the start of the step
    (``ModelSpec.keep_embedding``), ``step`` ``[passes, d]``.  ``spec.extra``: ``width``, ``passes``, ``names`` (the
    two tensors); the number of the pass is the layer call's ``arg``.  It has no cache."""
    graph_safe = True

    def __init__(self, env, spec):
        from .base import PartSpec
        self.env = env
        ex = spec.extra
        self.d, self.passes = int(ex["width"]), int(ex["passes"])
        self.mixer = None
        self.w = self.step = None
        self._inner = _ReentryTensors(self)
        self.children = (("reentry", self._inner, PartSpec("reentry", {}, dict(ex["names"]))),)
        self.step_arrays = ()

    def cache_needs(self):
        return {}

    def forward(self, h, pending, ctx, cache):
        from ..csrc import hipops
        from .linear import linear
        T, d, ws = h.shape[0], self.d, ctx.ws
        h0 = ctx.extras.get("h0")
        if h0 is None:
            raise ValueError("reentry: the model spec does not keep the embedding's result (keep_embedding)")
        d1, d2 = two_increments(h, pending)                 # everything still on its way joins the stream first
        if d1 is not None:
            hipops.add_into(h, d1[:T])
        if d2 is not None:
            hipops.add_into(h, d2[:T])
        both = ws.take((T, 2 * d), self.env.dtype)
        hipops.concat_rows(h, h0, both)
        y = ws.take((T, d), torch.float32)
        linear(both, self.w, y, ws=ws)
        which = int(ctx.extras["call"].arg or 0)
        if not 0 <= which < self.passes:
            raise ValueError(f"reentry: pass {which} of {self.passes}")
        hipops.bias_rows(y, self.step[which], h)
        return ()

    def stages(self):
        def whole(state, ctx, cache):
            ctx.extras["h0"] = state.get("h0")
            state["pending"] = self.forward(state["h"], state["pending"], ctx, cache)
        return [(True, whole)]


class _ReentryTensors:
    """The tensors of a ``reentry`` block, as the loader sees a part."""
    graph_safe = True
    step_arrays = ()

    def __init__(self, block):
        self.block = block

    def params(self):
        from .base import ParamSpec
        b = self.block
        return {"mix": ParamSpec((b.d, 2 * b.d)), "step": ParamSpec((b.passes, b.d), kind="vector", init="normal")}

    def load(self, t):
        from .linear import Weight
        b = self.block
        b.w = Weight(t["mix"])
        b.step = t["step"].float().contiguous()

    def slow_paths(self, page_size):
        return self.block.w.slow_reason("reentry matrix") if self.block.w is not None else []
