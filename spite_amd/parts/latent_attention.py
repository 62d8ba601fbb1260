"""Latent attention over the paged cache.

Every position caches one row: a latent vector c (``kv_rank`` elements, RMS-normed with a
weight) and one rotated key part (``rot_dim`` elements) that all heads share.  Head h's key at a
position is [U_h c | rotated part], its value V_h c.  The per-head matrices are folded into the
query and the result instead of being applied to cached rows:

    score_h(i, j) = (U_h^T a_h(i)) . c_j + b_h(i) . k_j        (query of head h = [a_h | b_h])
    out_h(i)      = V_h (sum_j softmax_j(score_h(i, .) * scale) c_j)

so the attention kernel sees one shared kv head whose rows are ``kv_rank + rot_dim`` wide and whose
value is the row's first ``kv_rank`` elements.  The two per-head products run as grouped products
with one group a head over a row list (rows lie token by token, groups want them head by head).

A layer may read the rows that an earlier layer cached (``own_kv=False``): it has no
down-projection, but queries, per-head matrices, mask and output projection of its own.
"""
from __future__ import annotations

import torch

from .base import Mixer, ParamSpec, CacheNeed, KVNeed, register, register_step_array, build as build_part
from .linear import linear, Weight
from ..csrc import hipops


def _workgroups_name(H: int) -> str:
    """The step array with the MFMA kernel's work list for models of H heads (registered on demand:
    the list depends on the step's entries and on H alone)."""
    name = f"latent_attention.workgroups/{H}"
    register_step_array(name, lambda host: hipops.latent_workgroups(host.counts, host.cu_seqlens, H))
    return name


@register("mixer", "latent_attention")
class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, env, hidden_size, n_heads, dim, rot_dim, v_dim, kv_rank, scale, position, norm_eps,
                 visibility="full", span=0, own_kv=True, cache_visibility=None, cache_span=None):
        """``dim`` / ``rot_dim``: unrotated / rotated query and key elements of a head; ``v_dim``: a head's
        value; ``kv_rank``: the latent.  ``position``: the encoding of the rotated parts (its frequency
        table; adjacent pairs).  ``visibility`` / ``span``: what this layer's queries read;
        ``cache_visibility`` / ``cache_span``: what the cache must keep (the widest of all layers that
        read it; default: this layer's own)."""
        if visibility not in hipops.VIS:
            raise ValueError(f"latent attention: visibility {visibility!r} (known: {sorted(hipops.VIS)})")
        if visibility != "full" and span < 1:
            raise ValueError(f"latent attention: {visibility} of size {span}")
        self.env = env
        self.d, self.H, self.n, self.r = int(hidden_size), int(n_heads), int(dim), int(rot_dim)
        self.v, self.R = int(v_dim), int(kv_rank)
        self.Dk = self.R + self.r
        self.scale, self.eps = float(scale), float(norm_eps)
        self.visibility, self.span = visibility, int(span or 0)
        self.cache_visibility = cache_visibility or visibility
        self.cache_span = int(cache_span if cache_span is not None else self.span)
        self.own = bool(own_kv)
        self.position = build_part("position", position, env)
        if self.position.kernel_args().get("magnitude", 1.0) != 1.0:
            raise ValueError("latent_attention: a position encoding that scales sine and cosine is not what this mixer's kernel applies")
        ka = self.position.kernel_args()
        if self.r and not (ka.get("use_rope") and ka.get("adjacent")):
            raise ValueError("latent attention: the rotated parts take a rotary encoding with adjacent pairs")
        self.inv_freq = ka["inv_freq"]
        self.rot_dims = int(ka.get("rotary_dim") or 0)
        if self.rot_dims > self.r:
            raise ValueError(f"latent attention: {self.rot_dims} turning elements of a rotated part of {self.r}")
        self.wq = self.wdkv = self.w_norm = self.w_absorb = self.w_up = self.wo = None
        self.mfma = env.dtype == torch.bfloat16 and hipops.attn_latent_mfma_ok(self.Dk, self.R, 0)
        self._wg = _workgroups_name(self.H) if self.mfma else None
        self.step_arrays = (self._wg,) if self.mfma else ()

    def params(self):
        d, H, n, r, v, R = self.d, self.H, self.n, self.r, self.v, self.R
        p = {"q": ParamSpec((H * (n + r), d)), "uk": ParamSpec((H * n, R)), "uv": ParamSpec((H * v, R)),
             "o": ParamSpec((d, H * v))}
        if self.own:
            p["dkv"] = ParamSpec((R + r, d))
            p["dkv.norm"] = ParamSpec((R,), kind="vector", init="ones")
        return p

    def load(self, t):
        H, n, v, R = self.H, self.n, self.v, self.R
        self.wq = Weight(t["q"])
        if self.own:
            self.wdkv = Weight(t["dkv"])
            self.w_norm = t["dkv.norm"].contiguous()
        # U_h^T as a product's weight [out = R, in = n]; V_h is one already: [out = v, in = R]
        # (its input rows are column ranges of the query rows: operand order only if those stay aligned)
        self.w_absorb = Weight(t["uk"].view(H, n, R).transpose(1, 2).contiguous(), (n + self.r) % 8 == 0)
        self.w_up = Weight(t["uv"].view(H, v, R))
        self.wo = Weight(t["o"])

    def slow_paths(self, page_size):
        notes = []
        if self.env.dtype == torch.bfloat16:
            if not hipops.attn_latent_mfma_ok(self.Dk, self.R, page_size):
                notes.append(f"latent attention runs on plain FMAs: rows of {self.Dk} with a latent of {self.R} "
                             f"(the MFMA kernel takes multiples of 8, rows up to 576, latents up to 512)")
            for name, w in (("query projection", self.wq), ("down-projection", self.wdkv), ("per-head key matrices", self.w_absorb),
                            ("per-head value matrices", self.w_up), ("output projection", self.wo)):
                if w is not None:
                    notes += w.slow_reason(name)
        return notes

    def cache_need(self):
        if not self.own:
            return CacheNeed()
        # one kv head; the value is part of the key row, so the pool's value half is empty
        return CacheNeed(kv=KVNeed(1, self.Dk, self.cache_visibility, self.cache_span, v_head_dim=0))

    def forward(self, x, ctx, cache):
        T = x.shape[0]
        H, n, r, v, R, Dk = self.H, self.n, self.r, self.v, self.R, self.Dk
        ws = ctx.ws
        q = ws.take((T, H * (n + r)), x.dtype)
        linear(x, self.wq, q, ws=ws)
        dkv = None
        if self.own:
            if not cache.write:
                raise RuntimeError("latent attention: a layer with a down-projection of its own must write its cache")
            dkv = ws.take((T, R + r), x.dtype)
            linear(x, self.wdkv, dkv, ws=ws)
        qa = ws.take((T * H, Dk), x.dtype)
        rows_th, offsets_h = ws.take((H * T,), torch.int32), ws.take((H + 1,), torch.int32)
        hipops.latent_prepare(q, dkv, qa, cache.k_pages, ctx.positions, cache.slot_map, self.inv_freq, self.w_norm,
                              self.eps, H, n, r, R, self.rot_dims, self.own, rows_th, offsets_h)
        # U_h^T a_h into the first R elements of every query row: one group a head
        linear(q.view(T * H, n + r)[:, :n], self.w_absorb, qa[:, :R], offsets=offsets_h, n_groups=H, a_rows=rows_th,
               y_rows=rows_th, rows=H * T, max_rows=T, ws=ws)
        o_lat = ws.take((T * H, R), x.dtype)
        if self.mfma:
            wg, (n_wg, most) = ctx.derived[self._wg]
            # the most keys that a query of the step may read, bounded by the block table's width (the same
            # for every step of one shape) and by the layer's reach
            longest = cache.block_table.shape[1] * cache.page_size
            if self.visibility != "full":
                longest = min(longest, self.span + ctx.max_count + 31)
            n_splits = hipops.latent_splits(n_wg, longest)
            scratch = ws.take((T * H * n_splits * (R + 2),), torch.float32) if n_splits > 1 else None
            hipops.attn_latent_mfma(qa, cache.k_pages, o_lat, ctx.positions, ctx.seq_of_token, cache.block_table,
                                    wg, n_wg, most, T, H, Dk, R, self.visibility, self.span, self.scale,
                                    n_splits=n_splits, scratch=scratch)
        else:
            hipops.attn_latent_generic(qa, cache.k_pages, o_lat, ctx.positions, ctx.seq_of_token, cache.block_table,
                                       T, H, Dk, R, self.visibility, self.span, self.scale)
        o = ws.take((T, H * v), x.dtype)
        linear(o_lat, self.w_up, o.view(T * H, v), offsets=offsets_h, n_groups=H, a_rows=rows_th, y_rows=rows_th,
               rows=H * T, max_rows=T, ws=ws)
        out = ws.take((T, self.d), torch.float32)
        linear(o, self.wo, out, ws=ws)
        return out
