"""ctypes binding of the gfx950 kernel library: one Python function per entry point.

Arguments are torch tensors on the GPU; each wrapper checks device, dtype, contiguity and the
shapes that the kernel's indexing assumes before it launches, and raises ``KernelError`` with
the library's message when the library refuses a size.  There is no fallback: without the
library, or with a tensor that is not on the GPU, the call fails.
"""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_long, c_float, c_void_p, c_size_t, c_char_p

import numpy as np
import torch

from . import build

F32, BF16 = 0, 1
VIS = build.visibility_codes()      # "full", "chunk", "window": name -> code
# the gate's activation of a gated product act(gate) * up, as the kernels number them (True: silu)
GATE_ACTS = {False: 0, None: 0, True: 1, "silu": 1, "gelu_tanh": 2, "relu": 3}
# an activation of a plain product's own (no gate), as the kernels number them; the bf16 weight-stream and
# tiled products take it in their epilogue, in the bits above the gate's code
UNARY_ACTS = {"gelu": 1, "gelu_tanh": 2, "silu": 3, "tanh": 4}


class KernelError(RuntimeError):
    pass


_lib = None


def lib():
    global _lib
    if _lib is None:
        l = build.load("hip")
        l.spite_hip_last_error.restype = c_char_p
        P, I, L, F = c_void_p, c_int, c_long, c_float
        sigs = {
            "spite_embed": [P, P, I, P, I, I, I, F, P],
            "spite_add_rmsnorm": [P, P, P, P, P, I, P, P, I, I, F, I, P, P, I, P, P, F, F, I, P, P, P],
            "spite_rope_kvwrite": [P, P, P, P, I, P, P, P, I, I, I, I, I, I, I, I, F, I, I, F, I, I, I, P, P, I, P],
            "spite_router_top1": [P, P, P, P, P, I, I, I, P],
            "spite_moe_plan": [P, P, P, P, P, P, P, I, I, I, I, P],
            "spite_convert": [P, I, P, I, c_size_t, P],
            "spite_add_into": [P, P, c_size_t, P],
            "spite_randn_fill": [P, I, c_size_t, ctypes.c_ulonglong, ctypes.c_ulonglong, F, F, P],
            "spite_gemm_generic": [P, I, P, L, I, P, I, I, I, I, I, P, I, P, P, P, I, P],
            "spite_attn_generic": [P, P, P, P, I, P, P, P, I, I, I, I, I, I, I, I, F, F, P, I, P],
            "spite_sample_rows": [P, I, I, I, P, P, P, P],
            "spite_filter_rows": [P, I, I, I, P, P, P, P],
            "spite_gemm_skinny": [P, I, P, L, P, I, I, I, I, I, P, I, P, P, P, I, I, I, I, I, P],
            "spite_attn_decode": [P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, F, F, P, I, I, P, P],
            "spite_gemm_mfma": [P, I, P, L, P, I, I, I, I, I, P, I, P, P, P, I, I, P],
            "spite_gemm_tiled": [P, I, P, L, P, I, I, I, I, I, P, I, P, P, P, I, I, P],
            "spite_gemm_tiled_split": [P, I, P, P, I, I, I, I, I, I, P, P],
            "spite_attn_prefill": [P, P, P, P, P, P, P, P, I, P, I, I, I, I, I, I, I, F, F, P, I, I, P, P],
            "spite_attn_prefill_splits": [P, I, I, I, L],
            "spite_argmax_rows": [P, I, I, I, P, P, P, P],
            "spite_stream_read": [P, c_size_t, P, I, P],
            "spite_mfma_loop": [P, I, I, F, P],
            "spite_latent_prepare": [P, I, P, I, P, P, I, P, P, P, P, F, I, I, I, I, I, I, I, P, P, P],
            "spite_attn_latent_generic": [P, P, P, I, P, P, P, I, I, I, I, I, I, I, I, F, P],
            "spite_attn_latent_mfma": [P, P, P, P, P, P, I, P, I, I, I, I, I, I, I, I, F, P, I, I, P],
            "spite_router_topk": [P, P, P, P, I, I, I, I, I, P],
            "spite_moe_combine": [P, P, P, P, I, I, I, P],
            "spite_gated_rows": [P, I, P, P, I, I, I, P, I, I, P],
            "spite_qkv_prepare": [P, I, I, P, P, P, F, P, P, P, P, P, P, I, F, P, I, I, I, I, I, I, I, I, I, I, I, F, I, I, P],
            "spite_attn_wide": [P, P, P, P, I, I, P, P, P, I, I, I, I, I, I, I, I, I, I, F, I, I, P, P, P],
            "spite_attn_finish": [P, I, P, I, P, P, P, I, I, I, I, I, F, F, F, P],
            "spite_token_shift": [P, P, I, P, P, P, P, P, I, I, I, P],
            "spite_act_rows": [P, I, c_size_t, I, P],
            "spite_scale_rows": [P, c_size_t, F, P],
            "spite_channel_decay": [P, P, I, I, F, I, P],
            "spite_linear_attn_scan": [P, P, P, I, I, I, I, P, P, F, P, I, P, P, I, P, I, I, I, I, I, I, P, P, P],
            "spite_gated_group_norm": [P, P, I, P, I, P, I, I, I, I, F, I, I, P, I, P, I, P],
            "spite_add_tanh_norm": [P, P, P, P, P, P, P, F, P, P, P, P, I, P, P, I, I, I, P],
            "spite_add_tanh_norm_proj": [P, P, P, P, P, P, P, F, P, P, P, P, I, P, I, I, I, P, P, I, P],
            "spite_hash_rows": [P, P, P, P, P, P, P, I, ctypes.c_longlong, ctypes.c_longlong, ctypes.c_longlong, I, P],
            "spite_embed_sum": [P, P, P, P, I, P, I, I, I, I, F, P],
            "spite_causal_conv": [P, I, I, P, P, P, P, P, P, I, P, I, I, I, I, I, I, I, P],
            "spite_shift_mix": [P, I, P, P, P, P, P, P, I, I, I, I, P],
            "spite_step_decay": [P, I, I, P, P, P, P, I, I, I, P],
            "spite_softcap_rows": [P, c_size_t, F, P],
            "spite_axpby_rows": [P, P, P, c_size_t, F, F, P],
            "spite_concat_rows": [P, P, P, I, I, I, P],
            "spite_bias_rows": [P, P, P, I, I, P],
        }
        for name, args in sigs.items():
            fn = getattr(l, name)
            fn.argtypes = args
            fn.restype = c_int
        l.spite_attn_prefill_workspace.argtypes = [P, I, I, I, I, I]
        l.spite_attn_prefill_workspace.restype = c_size_t
        l.spite_cu_count.argtypes = []
        l.spite_cu_count.restype = c_int
        _lib = l
    return _lib


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise KernelError(f"no kernel for dtype {dt}; the engine computes in float32 or bfloat16")


def _ptr(t, name, dtype=None, optional=False):
    if t is None:
        if optional:
            return None
        raise KernelError(f"{name}: missing tensor")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on {t.device}; the kernels run on the GPU only")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    return t.data_ptr()


def _ptr_rows(t, name):
    """A matrix whose rows may lie apart (a column range of a wider one): the products take the
    row stride beside the pointer."""
    if t is not None and t.dim() == 2 and t.is_cuda and t.stride(1) == 1 and t.stride(0) >= t.shape[1]:
        return t.data_ptr()
    return _ptr(t, name)


def _check_pages(k_pages, v_pages, G, page_size, hd, what, value_heads=None):
    """Key pages [n, G, page_size, hd]; value pages transposed, [n, G (or value_heads), hd, page_size]."""
    if (tuple(k_pages.shape[1:]) != (G, page_size, hd) or tuple(v_pages.shape[1:]) != (value_heads or G, hd, page_size)
            or k_pages.shape[0] != v_pages.shape[0]):
        raise KernelError(f"{what}: key pages {tuple(k_pages.shape)}, value pages {tuple(v_pages.shape)} for "
                          f"G={G} page={page_size} hd={hd}")


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _check(rc, what):
    if rc != 0:
        raise KernelError(f"{what}: {lib().spite_hip_last_error().decode()}")


# --------------------------------------------------------------------------------------------
def embed(ids, table, h, scale=1.0):
    """h[t,:] = table[ids[t],:] * scale as fp32.  ids int32 [T], table [V,d], h fp32 [T,d]."""
    T, d = h.shape
    if ids.numel() != T or table.shape[1] != d:
        raise KernelError(f"embed: ids {tuple(ids.shape)}, table {tuple(table.shape)}, h {tuple(h.shape)}")
    _check(lib().spite_embed(_ptr(ids, "ids", torch.int32), _ptr(table, "table"), dtype_code(table.dtype),
                             _ptr(h, "h", torch.float32), T, d, table.shape[0], float(scale), _stream()), "embed")


def add_rmsnorm_can_project(d: int) -> bool:
    """Whether ``add_rmsnorm`` forms projections of rows of this width (the row stays in LDS)."""
    return d * 4 <= 48 * 1024


def add_rmsnorm(h, w, eps, out=None, out32=None, d1=None, d2=None, rows=None, n_rows=None, write_h=True,
                proj=None, proj_out=None, normed=None, plain_out=False, w2=None, out2=None):
    """v = h[r] + d1[r] + d2[r] (stored back if write_h); out[i] = rmsnorm(v) * w with r =
    rows[i] or i.  h, d1, d2, out32 fp32; w fp32 [d]; out fp32 or bf16.  With ``proj`` ([P, d]
    fp32) also proj_out[i] = proj . (the normed row in fp32), [n, P] fp32: the same bits as
    ``router_top1`` gives for that row.  ``normed`` = (dn, wn, mult, eps_n): a further increment
    mult * rmsnorm(dn[r]; eps_n) * wn, normed on its way in.  ``plain_out``: out[i] = v itself (no
    norm; ``w`` may be None).  ``w2`` / ``out2``: the same rows normed with a second weight (in the
    dtype of ``out`` where there is one).  With no output at all the call only adds."""
    d = h.shape[-1]
    dn = wn = None
    mult = eps_n = 0.0
    if normed is not None:
        dn, wn, mult, eps_n = normed
        if dn.shape[-1] != d or dn.shape[0] < h.shape[0] or wn.numel() != d:
            raise KernelError(f"add_rmsnorm: normed increment {tuple(dn.shape)} with weight of {wn.numel()} for h {tuple(h.shape)}")
    if w is None and not plain_out and (out is not None or out32 is not None or proj is not None):
        raise KernelError("add_rmsnorm: a normed output needs the norm's weight")
    n = n_rows if n_rows is not None else (rows.numel() if rows is not None else h.shape[0])
    for name, t in (("d1", d1), ("d2", d2)):
        if t is not None and (t.shape[-1] != d or t.shape[0] < h.shape[0]):
            raise KernelError(f"add_rmsnorm: {name} {tuple(t.shape)} does not match h {tuple(h.shape)}")
    if w is not None and w.numel() != d:
        raise KernelError(f"add_rmsnorm: weight of {w.numel()} for rows of {d}")
    if out2 is not None and (w2 is None or w2.numel() != d or (out is not None and out2.dtype != out.dtype)):
        raise KernelError("add_rmsnorm: the second output needs a weight of its own and the first output's dtype")
    for name, t in (("out", out), ("out32", out32), ("out2", out2)):
        if t is not None and (t.shape[-1] != d or t.shape[0] < n):
            raise KernelError(f"add_rmsnorm: {name} {tuple(t.shape)} is too small for {n} rows of {d}")
    if rows is None and n > h.shape[0]:
        raise KernelError("add_rmsnorm: more rows asked than h holds")
    P = 0
    if proj is not None:
        P = proj.shape[0]
        if proj.dim() != 2 or proj.shape[1] != d or proj_out is None or proj_out.dim() != 2 \
                or proj_out.shape[0] < n or proj_out.shape[1] != P:
            raise KernelError("add_rmsnorm: projection [P, d] with an output [rows, P]")
    _check(lib().spite_add_rmsnorm(
        _ptr(h, "h", torch.float32), _ptr(d1, "d1", torch.float32, True), _ptr(d2, "d2", torch.float32, True),
        _ptr(w, "w", torch.float32, True), _ptr(out, "out", None, True),
        dtype_code(out.dtype) if out is not None else (dtype_code(out2.dtype) if out2 is not None else F32),
        _ptr(out32, "out32", torch.float32, True),
        _ptr(rows, "rows", torch.int32, True), n, d, float(eps), int(write_h),
        _ptr(proj, "proj", torch.float32, True), _ptr(proj_out, "proj_out", torch.float32, True), P,
        _ptr(dn, "normed increment", torch.float32, True), _ptr(wn, "normed increment's weight", torch.float32, True),
        float(mult), float(eps_n), int(bool(plain_out)), _ptr(w2, "w2", torch.float32, True), _ptr(out2, "out2", None, True),
        _stream()),
        "add_rmsnorm")


def rope_kvwrite(qkv, q_out, k_pages, v_pages, positions, slot_map, inv_freq, H, G, hd, page_size, *,
                 use_rope, adjacent, use_norm, norm_eps, use_temp, floor_scale, attn_scale, write_kv=True,
                 kv_tiled=False, rotary_dim=None, norm_weight_q=None, norm_weight_k=None, norm_first=False):
    """Rotation, qk-norm and temperature of the fused projection's rows; keys and values go to
    their cache rows.  qkv [T,(H+2G)*hd]; q_out [T,H*hd]; key pages [n_pages, G, page_size, hd],
    value pages [n_pages, G, hd, page_size].  ``rotary_dim``: only the first so many elements of a
    head rotate (default: all); ``norm_weight_q`` / ``norm_weight_k`` (fp32 [hd]): the norm's
    weights (default: weightless); ``norm_first``: the norm comes before the rotation."""
    T = qkv.shape[0]
    if qkv.shape[1] != (H + 2 * G) * hd:
        raise KernelError(f"rope_kvwrite: qkv {tuple(qkv.shape)} for H={H} G={G} hd={hd}")
    if q_out.numel() < T * H * hd or positions.numel() < T:
        raise KernelError("rope_kvwrite: q_out or positions too small")
    if write_kv:
        if slot_map.numel() < T:
            raise KernelError("rope_kvwrite: slot map too small")
        _check_pages(k_pages, v_pages, G, page_size, hd, "rope_kvwrite")
    rot = hd if rotary_dim is None else int(rotary_dim)
    if hd % 2:
        raise KernelError(f"rope_kvwrite: head size {hd} must be even")
    if rot % 2 or not 0 < rot <= hd:
        raise KernelError(f"rope_kvwrite: {rot} rotating elements of a head of {hd}")
    if use_rope and inv_freq.numel() != rot // 2:
        raise KernelError("rope_kvwrite: frequency table does not match the rotating part of the head")
    for name, w in (("norm_weight_q", norm_weight_q), ("norm_weight_k", norm_weight_k)):
        if w is not None and (w.numel() != hd or not use_norm):
            raise KernelError(f"rope_kvwrite: {name} of {w.numel()} for heads of {hd} (norm {'on' if use_norm else 'off'})")
    dt = qkv.dtype
    _check(lib().spite_rope_kvwrite(
        _ptr(qkv, "qkv"), _ptr(q_out, "q_out", dt), _ptr(k_pages, "k_pages", dt, not write_kv),
        _ptr(v_pages, "v_pages", dt, not write_kv), dtype_code(dt), _ptr(positions, "positions", torch.int32),
        _ptr(slot_map, "slot_map", torch.int32, not write_kv), _ptr(inv_freq, "inv_freq", torch.float32, not use_rope),
        T, H, G, hd, page_size, int(use_rope), int(adjacent), int(use_norm), float(norm_eps), int(use_temp),
        int(floor_scale), float(attn_scale), int(write_kv), int(bool(kv_tiled)), rot,
        _ptr(norm_weight_q, "norm_weight_q", torch.float32, True), _ptr(norm_weight_k, "norm_weight_k", torch.float32, True),
        int(bool(norm_first)), _stream()), "rope_kvwrite")


def router_top1(x32, w_router, expert, weight, logits_out=None):
    """Top-1 sigmoid router on fp32 rows.  x32 [T,d], w_router fp32 [E,d]."""
    T, d = x32.shape
    E = w_router.shape[0]
    if w_router.shape[1] != d or expert.numel() < T or weight.numel() < T:
        raise KernelError("router_top1: shapes do not match")
    if logits_out is not None and logits_out.numel() < T * E:
        raise KernelError("router_top1: logits_out too small")
    _check(lib().spite_router_top1(_ptr(x32, "x32", torch.float32), _ptr(w_router, "w_router", torch.float32),
                                   _ptr(expert, "expert", torch.int32), _ptr(weight, "weight", torch.float32),
                                   _ptr(logits_out, "logits_out", torch.float32, True), T, d, E, _stream()),
           "router_top1")


def moe_plan(expert, weight, src, scale, dst, offsets, T, E, shared, logits=None, fan=1):
    """Row list of the grouped products from the router's choice (see the kernel).  With
    ``logits`` ([T, E] fp32) the choice is made here and written to ``expert`` and ``weight``.
    ``fan`` > 1: the T entries are ``fan`` choices in a row for each of T / fan tokens; ``src`` names
    the token (entry // fan), ``dst`` the entry."""
    n = 2 * T if shared else T
    if src.numel() < n or scale.numel() < n or dst.numel() < n or offsets.numel() < E + 1 + int(bool(shared)):
        raise KernelError("moe_plan: output arrays too small")
    if expert.numel() < T or weight.numel() < T:
        raise KernelError("moe_plan: inputs too small")
    if logits is not None and (logits.dim() != 2 or logits.shape[0] < T or logits.shape[1] != E):
        raise KernelError(f"moe_plan: logits {tuple(logits.shape)} for {T} tokens and {E} experts")
    _check(lib().spite_moe_plan(_ptr(expert, "expert", torch.int32), _ptr(weight, "weight", torch.float32),
                                _ptr(logits, "logits", torch.float32, True), _ptr(src, "src", torch.int32), _ptr(scale, "scale", torch.float32),
                                _ptr(dst, "dst", torch.int32), _ptr(offsets, "offsets", torch.int32),
                                T, E, int(bool(shared)), int(fan), _stream()), "moe_plan")


def convert(src, dst):
    if src.numel() != dst.numel():
        raise KernelError("convert: sizes differ")
    _check(lib().spite_convert(_ptr(src, "src"), dtype_code(src.dtype), _ptr(dst, "dst"), dtype_code(dst.dtype),
                               src.numel(), _stream()), "convert")


def add_into(h, d):
    """h += d, both fp32 and of one size (an increment of the residual stream beyond the two
    that a norm adds itself)."""
    if h.numel() != d.numel() or not h.is_contiguous() or not d.is_contiguous():
        raise KernelError(f"add_into: {tuple(h.shape)} and {tuple(d.shape)} must be contiguous and of one size")
    _check(lib().spite_add_into(_ptr(h, "h", torch.float32), _ptr(d, "d", torch.float32), h.numel(), _stream()), "add_into")


def randn_fill(t, seed: int, key: int, mean: float = 0.0, std: float = 1.0):
    """t[i] = mean + std * z(seed, key, i) with z standard normal: counter-based, so a tensor's
    numbers depend on the seed, its key and the element's index alone."""
    if not t.is_contiguous():
        raise KernelError("randn_fill: the tensor must be contiguous")
    _check(lib().spite_randn_fill(_ptr(t, "t"), dtype_code(t.dtype), t.numel(), int(seed) & ((1 << 64) - 1),
                                  int(key) & ((1 << 64) - 1), float(mean), float(std), _stream()), "randn_fill")


def gemm_generic(a, w, y, M, N, K, *, offsets=None, n_groups=1, a_rows=None, a_scale=None, y_rows=None,
                 glu=False):
    """Y = A . W^T (see gemm_generic.hip).  a [rows,K]; w [groups, N or 2N, K] or [N or 2N, K];
    y [rows,N]."""
    if a.shape[-1] != K or y.shape[-1] != N:
        raise KernelError(f"gemm: a {tuple(a.shape)}, y {tuple(y.shape)} for N={N} K={K}")
    rows_w = 2 * N if glu else N
    if w.shape[-1] != K or w.shape[-2] != rows_w:
        raise KernelError(f"gemm: weight {tuple(w.shape)} for N={N} K={K} glu={glu}")
    groups_w = w.shape[0] if w.dim() == 3 else 1
    if offsets is not None:
        if groups_w < n_groups or offsets.numel() < n_groups + 1:
            raise KernelError("gemm: fewer weight groups or offsets than groups")
    if a_rows is None and a.shape[0] < M:
        raise KernelError("gemm: A has fewer rows than M")
    if y_rows is None and y.shape[0] < M:
        raise KernelError("gemm: Y has fewer rows than M")
    for name, t in (("a_rows", a_rows), ("a_scale", a_scale), ("y_rows", y_rows)):
        if t is not None and t.numel() < M:
            raise KernelError(f"gemm: {name} shorter than M")
    if w.dtype != a.dtype:
        raise KernelError(f"gemm: activations {a.dtype} against weights {w.dtype}")
    _check(lib().spite_gemm_generic(
        _ptr_rows(a, "a"), a.stride(0) if a.dim() == 2 else K, _ptr(w, "w"), rows_w * K, dtype_code(a.dtype),
        _ptr_rows(y, "y"), dtype_code(y.dtype), y.stride(0), M, N, K, _ptr(offsets, "offsets", torch.int32, True), n_groups,
        _ptr(a_rows, "a_rows", torch.int32, True), _ptr(a_scale, "a_scale", torch.float32, True),
        _ptr(y_rows, "y_rows", torch.int32, True), int(glu), _stream()), "gemm")


def attn_generic(q, k_pages, v_pages, out, positions, seq_of_token, block_table, T, H, G, hd, page_size,
                 vis, span, scale, kv_tiled=False, softcap=0.0, slopes=None):
    """Attention over the paged cache, any mix of portions and single tokens.  q/out
    [T,H*hd]; block_table int32 [n_seqs, max_blocks].  ``kv_tiled``: the pages are in operand
    order (``kv_operand_order``).  Here and in the MFMA kernels: ``slopes`` (fp32 [H]) adds
    slopes[head] * (key position - query position) to the scaled scores; ``softcap`` > 0 then caps
    them smoothly, ``softcap * tanh(score / softcap)``, before the softmax."""
    if q.numel() < T * H * hd or out.numel() < T * H * hd:
        raise KernelError("attention: q or out too small")
    _check_pages(k_pages, v_pages, G, page_size, hd, "attention")
    if block_table.dim() != 2 or positions.numel() < T or seq_of_token.numel() < T:
        raise KernelError("attention: metadata too small")
    dt = q.dtype
    _check(lib().spite_attn_generic(
        _ptr(q, "q"), _ptr(k_pages, "k_pages", dt), _ptr(v_pages, "v_pages", dt), _ptr(out, "out", dt),
        dtype_code(dt), _ptr(positions, "positions", torch.int32), _ptr(seq_of_token, "seq_of_token", torch.int32),
        _ptr(block_table, "block_table", torch.int32), block_table.shape[1], T, H, G, hd, page_size,
        VIS[vis], int(span or 0), float(scale), float(softcap), _slopes(slopes, H), int(bool(kv_tiled)), _stream()), "attention")


def sample_rows(logits, temperature, uniform, out, n_rows=None):
    """out[r] = arg-max of row r (temperature[r] <= 0 or no temperatures) or the inverse-CDF
    draw with uniform[r].  logits fp32 [n,V]."""
    n = n_rows if n_rows is not None else logits.shape[0]
    if out.numel() < n or logits.shape[0] < n:
        raise KernelError("sample: too few rows")
    for name, t in (("temperature", temperature), ("uniform", uniform)):
        if t is not None and t.numel() < n:
            raise KernelError(f"sample: {name} shorter than the rows")
    _check(lib().spite_sample_rows(_ptr(logits, "logits", torch.float32), logits.stride(0), n, logits.shape[1],
                                   _ptr(temperature, "temperature", torch.float32, True),
                                   _ptr(uniform, "uniform", torch.float32, True),
                                   _ptr(out, "out", torch.int32), _stream()), "sample")


def filter_rows(work, params, pen_ids, pen_offsets):
    """The reference's filters on the rows of ``work`` (fp32 [n, V]) in place: repetition
    penalty, temperature, min-p, top-k, top-p (see sampling.hip).  ``params``: float64 [6, n]
    (on, temperature, ln(min_p), top_k, top_p, penalty); ``pen_ids`` int32, row r's distinct ids
    at ``pen_offsets[r] .. pen_offsets[r+1]`` (int32 [n+1]); the caller keeps the ids inside [0, V)."""
    n = work.shape[0]
    if params.dtype != torch.float64 or tuple(params.shape) != (6, n) or not params.is_contiguous():
        raise KernelError(f"filter: params {tuple(params.shape)} {params.dtype} for {n} rows")
    if pen_offsets.numel() != n + 1:
        raise KernelError(f"filter: {pen_offsets.numel()} offsets for {n} rows")
    _check(lib().spite_filter_rows(_ptr(work, "work", torch.float32), work.stride(0), n, work.shape[1],
                                   _ptr(params, "params", torch.float64), _ptr(pen_ids, "pen_ids", torch.int32, True),
                                   _ptr(pen_offsets, "pen_offsets", torch.int32), _stream()), "filter")


def _gemm_checks(a, w, y, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, what):
    if a.shape[-1] != K or y.shape[-1] != N:
        raise KernelError(f"{what}: a {tuple(a.shape)}, y {tuple(y.shape)} for N={N} K={K}")
    rows_w = 2 * N if glu else N
    if w.shape[-1] != K or w.shape[-2] != rows_w:
        raise KernelError(f"{what}: weight {tuple(w.shape)} for N={N} K={K} glu={glu}")
    groups_w = w.shape[0] if w.dim() == 3 else 1
    if offsets is not None and (groups_w < n_groups or offsets.numel() < n_groups + 1):
        raise KernelError(f"{what}: fewer weight groups or offsets than groups")
    if a_rows is None and a.shape[0] < M:
        raise KernelError(f"{what}: A has fewer rows than M")
    if y_rows is None and y.shape[0] < M:
        raise KernelError(f"{what}: Y has fewer rows than M")
    for name, t in (("a_rows", a_rows), ("a_scale", a_scale), ("y_rows", y_rows)):
        if t is not None and t.numel() < M:
            raise KernelError(f"{what}: {name} shorter than M")
    return rows_w


def gemm_skinny(a, w, y, M, N, K, *, offsets=None, n_groups=1, a_rows=None, a_scale=None, y_rows=None,
                glu=False, max_rows=None, variant=0, tiled=False, live_groups=0, act=None):
    """Weight-streaming bf16 product for few rows (see gemm_skinny.hip); arguments as gemm_generic.
    ``max_rows``: the most rows a group can bring (default M).  ``tiled``: w is in MFMA operand
    order (``operand_order``).  ``live_groups``: a promise that at most this many groups hold rows
    (0: none); row tiles beyond what that allows are not launched."""
    rows_w = _gemm_checks(a, w, y, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, "gemm_skinny")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"gemm_skinny: bfloat16 operands only, got {a.dtype} and {w.dtype}")
    _check(lib().spite_gemm_skinny(
        _ptr_rows(a, "a"), a.stride(0), _ptr(w, "w"), rows_w * K, _ptr_rows(y, "y"), dtype_code(y.dtype), y.stride(0),
        M, N, K, _ptr(offsets, "offsets", torch.int32, True), n_groups, _ptr(a_rows, "a_rows", torch.int32, True),
        _ptr(a_scale, "a_scale", torch.float32, True), _ptr(y_rows, "y_rows", torch.int32, True), _act_code(glu, act),
        int(max_rows if max_rows is not None else M), int(variant), int(bool(tiled)), int(live_groups), _stream()),
        "gemm_skinny")


def _act_code(glu, act) -> int:
    """The products' ``glu`` argument: the gate's code, or an activation of the product's own above it."""
    if act is None:
        return int(glu)
    if glu or act not in UNARY_ACTS:
        raise KernelError(f"product: activation {act!r} (known: {sorted(UNARY_ACTS)}; not beside a gate)")
    return UNARY_ACTS[act] << 4


def kv_tiled_ok(dtype, hd, page_size) -> bool:
    """Whether cache pages of this kind are kept in MFMA operand order."""
    return dtype == torch.bfloat16 and hd % 32 == 0 and page_size % 32 == 0


def kv_operand_order(k_pages, v_pages):
    """Copies of row-major pages (keys [n, G, page_size, hd], values transposed [n, G, hd,
    page_size]) in the operand order that the MFMA attention kernels read; same shapes.
    Keys: blocks of 32 keys, two tiles of 16 rows (row r of tile tt = key (r/4)*8 + tt*4 + r%4),
    hd/32 chunks each, a tile's [16 rows][32 elements] stored as [4 q][16 r][8 e].  Values:
    per block of 32 keys, tiles of 16 head elements, [16 rows][32 keys] stored the same way."""
    n, G, ps, hd = k_pages.shape
    if ps % 32 or hd % 32:
        raise KernelError(f"operand order needs page size {ps} and head size {hd} to be multiples of 32")
    # key offset w = 8a + 4tt + i  ->  row r = 4a + i of tile tt; element c = 32cc + 8q + e
    k = k_pages.reshape(n, G, ps // 32, 4, 2, 4, hd // 32, 4, 8)          # b, a, tt, i, cc, q, e
    k = k.permute(0, 1, 2, 4, 6, 7, 3, 5, 8)                                # b, tt, cc, q, a, i, e
    # head element c = 16dt + r, key offset = 32b + 8q + e
    Gv = v_pages.shape[1]                                                   # value heads may be fewer than key heads
    v = v_pages.reshape(n, Gv, hd // 16, 16, ps // 32, 4, 8)               # dt, r, b, q, e
    v = v.permute(0, 1, 4, 2, 5, 3, 6)                                      # b, dt, q, r, e
    return k.contiguous().view(n, G, ps, hd), v.contiguous().view(n, Gv, hd, ps)


def attn_decode_workspace(T, H, hd, n_splits) -> int:
    """Bytes of scratch that attn_decode needs."""
    return T * H * n_splits * (hd + 2) * 4


def attn_decode(q, k_pages, v_pages, out, workspace, positions, seq_of_token, block_table, T, H, G, hd,
                page_size, vis, span, scale, n_splits, softcap=0.0, slopes=None, value_heads=None, sinks=None):
    """Split-KV decode attention on MFMA (bf16; head sizes 64 and 128; pages of a multiple of 32
    keys, in operand order): every row of q is one query against its request's cache.
    ``value_heads``: the value pages hold fewer heads than the key pages (kv head g reads value
    head g % value_heads).  ``sinks`` (fp32 [H] or None): one more term exp(sinks[h]) in every
    softmax's denominator."""
    if q.dtype != torch.bfloat16:
        raise KernelError(f"attn_decode: bfloat16 only, got {q.dtype}")
    if q.numel() < T * H * hd or out.numel() < T * H * hd:
        raise KernelError("attn_decode: q or out too small")
    _check_pages(k_pages, v_pages, G, page_size, hd, "attn_decode", value_heads)
    if block_table.dim() != 2 or positions.numel() < T or seq_of_token.numel() < T:
        raise KernelError("attn_decode: metadata too small")
    if workspace.numel() * workspace.element_size() < attn_decode_workspace(T, H, hd, n_splits):
        raise KernelError("attn_decode: workspace too small")
    dt = torch.bfloat16
    _check(lib().spite_attn_decode(
        _ptr(q, "q", dt), _ptr(k_pages, "k_pages", dt), _ptr(v_pages, "v_pages", dt), _ptr(out, "out", dt),
        _ptr(workspace, "workspace"), _ptr(positions, "positions", torch.int32),
        _ptr(seq_of_token, "seq_of_token", torch.int32), _ptr(block_table, "block_table", torch.int32),
        block_table.shape[1], T, H, G, hd, page_size, VIS[vis], int(span or 0), float(scale), float(softcap),
        _slopes(slopes, H), int(n_splits), int(value_heads or 0), _slopes(sinks, H), _stream()), "attn_decode")


def gemm_mfma(a, w, y, M, N, K, *, offsets=None, n_groups=1, a_rows=None, a_scale=None, y_rows=None, glu=False,
              shape=0):
    """Tiled bf16 MFMA product for many rows (see gemm_mfma.hip); arguments as gemm_generic."""
    rows_w = _gemm_checks(a, w, y, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, "gemm_mfma")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"gemm_mfma: bfloat16 operands only, got {a.dtype} and {w.dtype}")
    _check(lib().spite_gemm_mfma(
        _ptr_rows(a, "a"), a.stride(0), _ptr(w, "w"), rows_w * K, _ptr_rows(y, "y"), dtype_code(y.dtype), y.stride(0),
        M, N, K, _ptr(offsets, "offsets", torch.int32, True), n_groups, _ptr(a_rows, "a_rows", torch.int32, True),
        _ptr(a_scale, "a_scale", torch.float32, True), _ptr(y_rows, "y_rows", torch.int32, True), int(glu),
        int(shape), _stream()), "gemm_mfma")


def operand_order(w: torch.Tensor) -> torch.Tensor:
    """A copy of the matrices ``w[..., N, K]`` (N % 16 == 0, K % 64 == 0) in MFMA operand order:
    tiles of 16 rows x 32 k, tile (i, j) at ((i * K/32) + j) * 512 elements, inside it
    W[16i + r][32j + 8q + e] at (q*16 + r) * 8 + e.  Shape and dtype stay as they are."""
    *lead, N, K = w.shape
    if N % 16 or K % 64:
        raise KernelError(f"operand order needs rows a multiple of 16 and columns of 64, got {N} x {K}")
    n = len(lead)
    t = w.reshape(*lead, N // 16, 16, K // 32, 4, 8).permute(*range(n), n, n + 2, n + 3, n + 1, n + 4)
    return t.contiguous().view(*lead, N, K)


def tiled_k_runs(M: int, N: int, K: int) -> int:
    """Into how many runs the tiled product cuts its sum over k: with tiles of 128 rows x 512
    columns for fewer than half of the chip's CUs, those are not filled, and a run keeps at least
    four steps of 64 k."""
    cus = cu_count()
    tiles = -(-M // 128) * -(-N // 512)
    steps = K // 64
    runs = min(8, cus // max(tiles, 1), steps // 4)
    while runs > 1 and -(-steps // runs) * (runs - 1) >= steps:      # no run may be empty
        runs -= 1
    return runs if tiles < cus // 2 and runs > 1 else 1


_cu_count = None


def cu_count() -> int:
    """Compute units of the current GPU, as the library counts them."""
    global _cu_count
    if _cu_count is None:
        _cu_count = int(lib().spite_cu_count())
    return _cu_count


def gemm_tiled(a, w, y, M, N, K, *, offsets=None, n_groups=1, a_rows=None, a_scale=None, y_rows=None, glu=False,
               shape=0, part=None, act=None):
    """Tiled bf16 MFMA product for many rows over weights in operand order (``operand_order``;
    see gemm_tiled.hip); arguments as gemm_generic.  ``part`` (fp32 ``[runs, M, N]``, plain
    products only): the sum over k is cut into ``runs`` runs, each a workgroup of its own, whose
    partial sums a second kernel adds: for few tiles (a short prompt against a narrow matrix),
    see ``tiled_k_runs``."""
    rows_w = _gemm_checks(a, w, y, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, "gemm_tiled")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"gemm_tiled: bfloat16 operands only, got {a.dtype} and {w.dtype}")
    if part is not None:
        if not (offsets is None and a_rows is None and a_scale is None and y_rows is None and not glu and shape == 0 and act is None):
            raise KernelError("gemm_tiled: partial sums are for plain products only")
        if part.dim() != 3 or part.shape[1] != M or part.shape[2] != N or part.shape[0] < 2 or part.shape[0] > 32 \
                or part.shape[0] * 2 > K // 64:
            raise KernelError(f"gemm_tiled: partial sums {tuple(part.shape)} for M={M} N={N} K={K}")
        _check(lib().spite_gemm_tiled_split(_ptr(a, "a"), a.stride(0), _ptr(w, "w"), _ptr(y, "y"), dtype_code(y.dtype),
                                            y.stride(0), M, N, K, part.shape[0], _ptr(part, "part", torch.float32),
                                            _stream()), "gemm_tiled")
        return
    _check(lib().spite_gemm_tiled(
        _ptr_rows(a, "a"), a.stride(0), _ptr(w, "w"), rows_w * K, _ptr_rows(y, "y"), dtype_code(y.dtype), y.stride(0),
        M, N, K, _ptr(offsets, "offsets", torch.int32, True), n_groups, _ptr(a_rows, "a_rows", torch.int32, True),
        _ptr(a_scale, "a_scale", torch.float32, True), _ptr(y_rows, "y_rows", torch.int32, True), _act_code(glu, act),
        int(shape), _stream()), "gemm_tiled")


def attn_prefill_splits(counts, H, G, max_keys) -> int:
    """Into how many splits the prefill kernel's tiles of this step are best cut (1: none), for
    ``counts`` query tokens per request and at most ``max_keys`` keys read by a query."""
    counts = np.ascontiguousarray(counts, dtype=np.int32)
    return int(lib().spite_attn_prefill_splits(counts.ctypes.data, int(counts.size), H, G, int(max_keys)))


def attn_prefill_workspace(counts, H, G, hd, n_splits) -> int:
    """Bytes of fp32 scratch that ``attn_prefill`` needs for ``n_splits`` > 1 (none for 1)."""
    counts = np.ascontiguousarray(counts, dtype=np.int32)
    return int(lib().spite_attn_prefill_workspace(counts.ctypes.data, int(counts.size), H, G, hd, int(n_splits)))


def attn_prefill(q, k_pages, v_pages, out, positions, cu_seqlens, counts, block_table,
                 H, G, hd, page_size, vis, span, scale, n_splits=1, scratch=None, softcap=0.0, slopes=None, value_heads=None,
                 sinks=None):
    """Prefill attention on MFMA (bf16; head sizes 64 and 128; pages of a multiple of 32 keys, in
    operand order).
    ``counts``: the number of query tokens of every request of the step, on the host, in the
    order of ``cu_seqlens`` (their running sum, on the device) and of the block table's rows.
    ``n_splits`` > 1 deals every tile's keys to that many workgroups; ``scratch`` (fp32,
    ``attn_prefill_workspace`` bytes) then holds their partial results.
    ``slopes`` (fp32 [H] or None): a bias slopes[head] * (key position - query position) on the
    scaled scores, before the cap.  ``sinks`` (fp32 [H] or None): one more term exp(sinks[h]) in
    every softmax's denominator."""
    if q.dtype != torch.bfloat16:
        raise KernelError(f"attn_prefill: bfloat16 only, got {q.dtype}")
    counts = np.ascontiguousarray(counts, dtype=np.int32)
    n_seqs = int(counts.size)
    T = int(counts.sum())
    if q.numel() < T * H * hd or out.numel() < T * H * hd:
        raise KernelError("attn_prefill: q or out too small")
    _check_pages(k_pages, v_pages, G, page_size, hd, "attn_prefill", value_heads)
    if block_table.dim() != 2 or block_table.shape[0] < n_seqs or positions.numel() < T:
        raise KernelError("attn_prefill: metadata too small")
    if cu_seqlens.numel() < n_seqs + 1:
        raise KernelError("attn_prefill: cu_seqlens shorter than the requests of the step")
    n_splits = int(n_splits)
    if n_splits > 1 and (scratch is None or scratch.numel() * 4 < attn_prefill_workspace(counts, H, G, hd, n_splits)):
        raise KernelError(f"attn_prefill: {n_splits} splits need {attn_prefill_workspace(counts, H, G, hd, n_splits)} bytes of scratch")
    dt = torch.bfloat16
    _check(lib().spite_attn_prefill(
        _ptr(q, "q", dt), _ptr(k_pages, "k_pages", dt), _ptr(v_pages, "v_pages", dt), _ptr(out, "out", dt),
        _ptr(scratch, "scratch", torch.float32) if n_splits > 1 else None,
        _ptr(positions, "positions", torch.int32), _ptr(cu_seqlens, "cu_seqlens", torch.int32),
        counts.ctypes.data, n_seqs, _ptr(block_table, "block_table", torch.int32), block_table.shape[1],
        H, G, hd, page_size, VIS[vis], int(span or 0), float(scale), float(softcap), _slopes(slopes, H), n_splits,
        int(value_heads or 0), _slopes(sinks, H), _stream()), "attn_prefill")


def _slopes(slopes, H):
    if slopes is None:
        return None
    if slopes.numel() != H:
        raise KernelError(f"score slopes: {slopes.numel()} values for {H} query heads")
    return _ptr(slopes, "slopes", torch.float32)


def argmax_rows(logits, out, scratch_v, scratch_i, n_rows=None):
    """out[r] = index of the largest logit of row r, the lowest among equals.  Scratch: 32 floats
    and 32 ints per row."""
    n = n_rows if n_rows is not None else logits.shape[0]
    if out.numel() < n or logits.shape[0] < n or scratch_v.numel() < 32 * n or scratch_i.numel() < 32 * n:
        raise KernelError("argmax: outputs or scratch too small")
    _check(lib().spite_argmax_rows(_ptr(logits, "logits", torch.float32), logits.stride(0), n, logits.shape[1],
                                   _ptr(scratch_v, "scratch_v", torch.float32), _ptr(scratch_i, "scratch_i", torch.int32),
                                   _ptr(out, "out", torch.int32), _stream()), "argmax")


def stream_read(t, out):
    """Reads the tensor ``t`` once with non-temporal loads, one contiguous piece per workgroup;
    ``out`` (fp32, eight elements per workgroup) receives sums that keep the loads alive.  For
    measuring the memory's read bandwidth."""
    nbytes = t.numel() * t.element_size()
    if out.numel() < 8:
        raise KernelError("stream_read: out holds eight floats per workgroup")
    _check(lib().spite_stream_read(_ptr(t, "t"), nbytes - nbytes % 16, _ptr(out, "out", torch.float32), out.numel() // 8,
                                   _stream()), "stream_read")


def mfma_loop(out, steps, gain):
    """Runs ``out.numel()`` workgroups of eight waves, every wave ``steps`` times 32 MFMA 16x16x32 on
    operands in registers (pseudo-random values scaled by ``gain``; 0: all zero): the matrix units'
    rate with nothing else moving.  Returns the flops done."""
    _check(lib().spite_mfma_loop(_ptr(out, "out", torch.float32), out.numel(), int(steps), float(gain), _stream()), "mfma_loop")
    return out.numel() * 8 * int(steps) * 32 * 16384


# -------------------------------------------------------------------------------------------- latent attention
def latent_prepare(qd, dkv, qa, kv_pages, positions, slot_map, inv_freq, w_norm, eps, H, n, r, R, rot_dims, own,
                   rows_th, offsets_h):
    """Between the projections and the per-head products of latent attention (see latent.hip):
    qd [T, H*(n+r)]; dkv [T, R+r] (with ``own``); qa [T*H, R+r] receives the rotated query parts; with ``own`` the
    cache row of every token (kv_pages [pages, 1, page_size, R+r]) receives the normed latent and the
    rotated shared key part; rows_th int32 [H*T] and offsets_h int32 [H+1] receive the row list of
    the per-head products."""
    T = qd.shape[0]
    Dk = R + r
    if qd.dim() != 2 or qd.stride(1) != 1 or qd.shape[1] < H * (n + r):
        raise KernelError(f"latent_prepare: qd {tuple(qd.shape)} for H={H} n={n} r={r} R={R} own={own}")
    if own and (dkv is None or dkv.dim() != 2 or dkv.stride(1) != 1 or dkv.shape[1] < R + r or dkv.shape[0] < T or dkv.dtype != qd.dtype):
        raise KernelError(f"latent_prepare: the down-projection's rows do not fit R={R} r={r}")
    if qa.numel() < T * H * Dk or positions.numel() < T or rows_th.numel() < H * T or offsets_h.numel() < H + 1:
        raise KernelError("latent_prepare: outputs or positions too small")
    if inv_freq.numel() < rot_dims // 2:
        raise KernelError("latent_prepare: frequency table shorter than the turning pairs")
    dt = qd.dtype
    if own:
        if kv_pages.dim() != 4 or kv_pages.shape[1] != 1 or kv_pages.shape[3] != Dk or slot_map.numel() < T or w_norm.numel() != R:
            raise KernelError(f"latent_prepare: pages {tuple(kv_pages.shape)} for rows of {Dk}, or slots / norm weight too small")
    _check(lib().spite_latent_prepare(
        _ptr_rows(qd, "qd"), qd.stride(0), _ptr_rows(dkv, "dkv") if own else None, dkv.stride(0) if own else 0, _ptr(qa, "qa", dt), _ptr(kv_pages, "kv_pages", dt, not own), dtype_code(dt),
        _ptr(positions, "positions", torch.int32), _ptr(slot_map, "slot_map", torch.int32, not own),
        _ptr(inv_freq, "inv_freq", torch.float32), _ptr(w_norm, "w_norm", torch.float32, not own), float(eps),
        T, H, n, r, R, int(rot_dims), int(bool(own)), _ptr(rows_th, "rows_th", torch.int32),
        _ptr(offsets_h, "offsets_h", torch.int32), _stream()), "latent_prepare")


def _latent_checks(q, kv_pages, out, positions, seq_of_token, block_table, T, H, Dk, R, what):
    if q.numel() < T * H * Dk or out.numel() < T * H * R:
        raise KernelError(f"{what}: q or out too small")
    if kv_pages.dim() != 4 or kv_pages.shape[1] != 1 or kv_pages.shape[3] != Dk:
        raise KernelError(f"{what}: pages {tuple(kv_pages.shape)} for rows of {Dk}")
    if block_table.dim() != 2 or positions.numel() < T or seq_of_token.numel() < T:
        raise KernelError(f"{what}: metadata too small")


def attn_latent_generic(q, kv_pages, out, positions, seq_of_token, block_table, T, H, Dk, R, vis, span, scale):
    """Attention of T*H query rows [Dk] over cache rows [Dk] whose first R elements are the value:
    one shared kv head, any mix of portions and single tokens.  out [T*H, R]."""
    _latent_checks(q, kv_pages, out, positions, seq_of_token, block_table, T, H, Dk, R, "latent attention")
    dt = q.dtype
    _check(lib().spite_attn_latent_generic(
        _ptr(q, "q"), _ptr(kv_pages, "kv_pages", dt), _ptr(out, "out", dt), dtype_code(dt),
        _ptr(positions, "positions", torch.int32), _ptr(seq_of_token, "seq_of_token", torch.int32),
        _ptr(block_table, "block_table", torch.int32), block_table.shape[1], T, H, Dk, R, kv_pages.shape[2],
        VIS[vis], int(span or 0), float(scale), _stream()), "latent attention")


# -------------------------------------------------------------------------------------------- several experts a token
ROUTER_SCORING = {"sigmoid": 0, "softmax_taken": 1}


def router_topk(logits, bias, expert, weight, top, renorm=False, scoring="sigmoid"):
    """From fp32 router logits [T, E]: scores sigmoid(z); the ``top`` experts with the largest
    score + bias (bias fp32 [E] or None; lowest index among equals) into expert[T*top], their
    scores (without the bias; divided by their sum with ``renorm``) into weight[T*top].  With
    ``scoring`` = ``softmax_taken`` the choice goes by z + bias and the weights are the softmax over the
    taken experts' logits."""
    T, E = logits.shape
    if scoring not in ROUTER_SCORING:
        raise KernelError(f"router_topk: scoring {scoring!r} (known: {sorted(ROUTER_SCORING)})")
    if expert.numel() < T * top or weight.numel() < T * top or (bias is not None and bias.numel() != E):
        raise KernelError("router_topk: outputs too small or bias of the wrong size")
    _check(lib().spite_router_topk(_ptr(logits, "logits", torch.float32), _ptr(bias, "bias", torch.float32, True),
                                   _ptr(expert, "expert", torch.int32), _ptr(weight, "weight", torch.float32),
                                   T, E, int(top), int(bool(renorm)), ROUTER_SCORING[scoring], _stream()), "router_topk")


def moe_combine(y, weight, extra, out, T, top):
    """out[t] = sum_j weight[t*top + j] * y[t*top + j] (+ extra[t]); all fp32; ``weight`` None: every weight 1."""
    d = out.shape[-1]
    if y.numel() < T * top * d or (weight is not None and weight.numel() < T * top) or out.numel() < T * d \
            or (extra is not None and extra.numel() < T * d):
        raise KernelError("moe_combine: arrays too small")
    _check(lib().spite_moe_combine(_ptr(y, "y", torch.float32), _ptr(weight, "weight", torch.float32, True),
                                   _ptr(extra, "extra", torch.float32, True), _ptr(out, "out", torch.float32),
                                   T, d, int(top), _stream()), "moe_combine")


def gated_rows(a, ids, table, col0, g):
    """g[t] = gelu_tanh(a[t]) * table[ids[t]][col0 : col0 + n]; a, g [T, n] in the run's dtype."""
    T, n = a.shape
    if g.numel() < T * n or ids.numel() < T or table.dim() != 2:
        raise KernelError("gated_rows: arrays too small")
    _check(lib().spite_gated_rows(_ptr(a, "a"), dtype_code(a.dtype), _ptr(ids, "ids", torch.int32), _ptr(table, "table"),
                                  dtype_code(table.dtype), table.shape[1], int(col0), _ptr(g, "g", a.dtype), T, n,
                                  _stream()), "gated_rows")


LATENT_WG_ROWS = 128      # query rows that one workgroup of the MFMA kernel takes at most


def attn_latent_mfma_ok(Dk, R, page_size) -> bool:
    """Whether the MFMA kernel of latent attention takes rows of Dk with a latent of R (bfloat16)."""
    return Dk % 8 == 0 and R % 8 == 0 and 0 < R <= 512 and R <= Dk <= 576


def latent_workgroups(counts, cu_seqlens, H):
    """The MFMA kernel's work list for a step: int32 pairs (first query row, rows), at most
    ``LATENT_WG_ROWS`` rows each and every pair inside one entry's rows (entry i holds the query rows
    cu[i]*H .. cu[i+1]*H), flat; and (pairs, the most rows of a pair)."""
    out = []
    most = 0
    for i, n in enumerate(counts):
        rows, r0 = int(n) * H, int(cu_seqlens[i]) * H
        for off in range(0, rows, LATENT_WG_ROWS):
            k = min(LATENT_WG_ROWS, rows - off)
            out += [r0 + off, k]
            most = max(most, k)
    return np.asarray(out, dtype=np.int32), (len(out) // 2, most)


def latent_splits(n_wg: int, longest: int) -> int:
    """Into how many workgroups the keys of every work item are best dealt, for ``n_wg`` items whose
    queries read at most ``longest`` keys: about one workgroup a compute unit, each with at least eight
    blocks of 32 keys (a workgroup's record is as large as what it reads of two or three such blocks)."""
    if n_wg <= 0:
        return 1
    # (no fewer than keep a share within the 4,096 keys whose cache rows the staging waves look up ahead)
    return max(1, min(-(-cu_count() // n_wg), -(-longest // 256), 256), min(-(-longest // 4096), 256))


def attn_latent_mfma(q, kv_pages, out, positions, seq_of_token, block_table, wg, n_wg, max_rows, T, H, Dk, R, vis, span, scale,
                     n_splits=1, scratch=None):
    """As ``attn_latent_generic`` on the matrix units (bfloat16; see ``attn_latent_mfma_ok``).  ``wg``:
    the work list of ``latent_workgroups`` on the device.  ``n_splits`` > 1 (``latent_splits``) deals
    every item's keys to that many workgroups; ``scratch`` (fp32, T*H*n_splits*(R+2) elements) then
    holds their records."""
    n_splits = int(n_splits)
    if n_splits > 1 and (scratch is None or scratch.dtype != torch.float32 or scratch.numel() < T * H * n_splits * (R + 2)):
        raise KernelError(f"latent attention (MFMA): {n_splits} splits need {T * H * n_splits * (R + 2)} floats of scratch")
    _latent_checks(q, kv_pages, out, positions, seq_of_token, block_table, T, H, Dk, R, "latent attention (MFMA)")
    if q.dtype != torch.bfloat16:
        raise KernelError(f"latent attention (MFMA): bfloat16 only, got {q.dtype}")
    if wg.numel() < 2 * n_wg or max_rows > LATENT_WG_ROWS:
        raise KernelError("latent attention (MFMA): work list too short or its pairs too long")
    dt = torch.bfloat16
    _check(lib().spite_attn_latent_mfma(
        _ptr(q, "q", dt), _ptr(kv_pages, "kv_pages", dt), _ptr(out, "out", dt), _ptr(positions, "positions", torch.int32),
        _ptr(seq_of_token, "seq_of_token", torch.int32), _ptr(block_table, "block_table", torch.int32),
        block_table.shape[1], _ptr(wg, "wg", torch.int32), int(n_wg), int(max_rows), H, Dk, R, kv_pages.shape[2],
        VIS[vis], int(span or 0), float(scale), _ptr(scratch, "scratch", torch.float32) if n_splits > 1 else None,
        n_splits, T * H, _stream()), "latent attention (MFMA)")


# -------------------------------------------------------------------------------------------- keys and values of unequal shape
def qkv_prepare(qkv, q_out, k_pages, v_pages, positions, slot_map, HQ, GK, GV, D, Vd, page_size, *, bias=None,
                norm_q=None, norm_k=None, eps=0.0, inv_freq=None, rot=0, inv_freq_v=None, write_kv=True,
                k_tiled=False, v_tiled=False, stored_dim=None, rot_magnitude=1.0, head_norm=False, q_temperature=None,
                values_from_keys=False):
    """Between a fused projection and the cache (see attn_wide.hip).  qkv: rows that begin with
    [HQ*D | GK*D | GV*Vd] (further columns are left alone); ``bias`` fp32 over those; ``norm_q`` /
    ``norm_k`` (fp32 [HQ*D], [GK*D]): weights of an RMS norm over the whole q and the whole k part;
    ``inv_freq`` (fp32 [rot/2]): the first ``rot`` elements of every q and k head turn in pairs
    (i, i + rot/2), sine and cosine times ``rot_magnitude``; ``inv_freq_v`` (fp32 [Vd/2]): the values turn in
    pairs (m, m + Vd/2).  q_out
    [T, HQ*Dp]; key pages [pages, GK, page_size, Dp]; value pages [pages, GV, Vd, page_size], with
    Dp = ``stored_dim`` (default D): queries and keys are stored that wide, zeros behind their D.
    ``head_norm``: ``norm_q`` / ``norm_k`` hold D weights each and every head is normed on its own.
    ``q_temperature`` = (coef, every): the queries (after their norm) times 1 + coef * ln(floor((p + 1) / every) + 1)
    at position p.  ``values_from_keys``: the row holds no values, [HQ*D | GK*D] only; the values are the keys as
    the row holds them, before norm and rotation (GV = GK, Vd = D)."""
    T = qkv.shape[0]
    Dp = int(stored_dim or D)
    n = (HQ + GK) * D + (0 if values_from_keys else GV * Vd)
    if values_from_keys and (GV != GK or Vd != D):
        raise KernelError("qkv_prepare: values taken from the keys have the keys' heads and width")
    qt_coef, qt_every = (float(q_temperature[0]), int(q_temperature[1])) if q_temperature else (0.0, 0)
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < n:
        raise KernelError(f"qkv_prepare: rows {tuple(qkv.shape)} for HQ={HQ} GK={GK} GV={GV} D={D} Vd={Vd}")
    if q_out.numel() < T * HQ * Dp or positions.numel() < T or Dp < D:
        raise KernelError("qkv_prepare: q_out or positions too small")
    if write_kv:
        if slot_map is None or slot_map.numel() < T:
            raise KernelError("qkv_prepare: slot map too small")
        if tuple(k_pages.shape[1:]) != (GK, page_size, Dp) or tuple(v_pages.shape[1:]) != (GV, Vd, page_size) \
                or k_pages.shape[0] != v_pages.shape[0]:
            raise KernelError(f"qkv_prepare: key pages {tuple(k_pages.shape)}, value pages {tuple(v_pages.shape)} for "
                              f"GK={GK} GV={GV} page={page_size} D={D} Vd={Vd}")
    for name, t, size in (("bias", bias, n), ("norm_q", norm_q, D if head_norm else HQ * D),
                          ("norm_k", norm_k, D if head_norm else GK * D),
                          ("inv_freq", inv_freq, rot // 2), ("inv_freq_v", inv_freq_v, Vd // 2)):
        if t is not None and t.numel() != size:
            raise KernelError(f"qkv_prepare: {name} of {t.numel()} values, expected {size}")
    if rot and inv_freq is None:
        raise KernelError("qkv_prepare: rotation needs a frequency table")
    dt = qkv.dtype
    _check(lib().spite_qkv_prepare(
        qkv.data_ptr() if qkv.is_cuda else _ptr(qkv, "qkv"), qkv.stride(0), dtype_code(dt), _ptr(bias, "bias", torch.float32, True),
        _ptr(norm_q, "norm_q", torch.float32, True), _ptr(norm_k, "norm_k", torch.float32, True), float(eps),
        _ptr(q_out, "q_out", dt), _ptr(k_pages, "k_pages", dt, not write_kv), _ptr(v_pages, "v_pages", dt, not write_kv),
        _ptr(positions, "positions", torch.int32), _ptr(slot_map, "slot_map", torch.int32) if write_kv else None,
        _ptr(inv_freq, "inv_freq", torch.float32, True), int(rot), float(rot_magnitude),
        _ptr(inv_freq_v, "inv_freq_v", torch.float32, True),
        T, HQ, GK, GV, D, Vd, page_size, int(bool(k_tiled)), int(bool(v_tiled)), Dp, int(bool(head_norm)), qt_coef, qt_every,
        int(bool(values_from_keys)), _stream()), "qkv_prepare")


def attn_wide(q, k_pages, v_pages, out, positions, seq_of_token, block_table, T, HQ, GK, GV, D, Vd, page_size, vis, span,
              scale, k_tiled=False, v_tiled=False, sinks=None, slopes=None):
    """Attention over the paged cache with keys of D and values of Vd elements, HQ query heads over
    GK key heads over GV value heads (query head h: key head h // (HQ/GK), value head of that % GV);
    any mix of portions and single tokens.  q [T, HQ*D]; out [T, HQ*Vd] in q's dtype or fp32.
    ``sinks`` (fp32 [HQ] or None): one more term exp(sinks[h]) in every softmax's denominator.
    ``slopes`` (fp32 [HQ] or None): slopes[h] * (key position - query position) is added to the scaled score."""
    if sinks is not None and sinks.numel() != HQ:
        raise KernelError(f"attention: {sinks.numel()} sinks for {HQ} query heads")
    if q.numel() < T * HQ * D or out.numel() < T * HQ * Vd:
        raise KernelError("attention: q or out too small")
    if tuple(k_pages.shape[1:]) != (GK, page_size, D) or tuple(v_pages.shape[1:]) != (GV, Vd, page_size) \
            or k_pages.shape[0] != v_pages.shape[0]:
        raise KernelError(f"attention: key pages {tuple(k_pages.shape)}, value pages {tuple(v_pages.shape)} for "
                          f"GK={GK} GV={GV} page={page_size} D={D} Vd={Vd}")
    if block_table.dim() != 2 or positions.numel() < T or seq_of_token.numel() < T:
        raise KernelError("attention: metadata too small")
    dt = q.dtype
    _check(lib().spite_attn_wide(
        _ptr(q, "q"), _ptr(k_pages, "k_pages", dt), _ptr(v_pages, "v_pages", dt), _ptr(out, "out"), dtype_code(dt),
        dtype_code(out.dtype), _ptr(positions, "positions", torch.int32), _ptr(seq_of_token, "seq_of_token", torch.int32),
        _ptr(block_table, "block_table", torch.int32), block_table.shape[1], T, HQ, GK, GV, D, Vd, page_size,
        VIS[vis], int(span or 0), float(scale), int(bool(k_tiled)), int(bool(v_tiled)),
        _ptr(sinks, "sinks", torch.float32, True), _slopes(slopes, HQ), _stream()), "attention")


def attn_finish(a, out, positions, H, Vd, *, maps=1, lam=0.0, eps=0.0, post=1.0, inv_freq_v=None, gate=None):
    """From the attention's result to the output projection's operand (see attn_wide.hip).  a
    [T, maps*H*Vd] (map by map), out [T, H*Vd].  ``maps`` = 2: a1 - lam * a2, divided by its root mean
    square over the head (``eps``), times ``post``.  ``inv_freq_v``: pairs (m, m + Vd/2) turn back by
    the position.  ``gate``: a [T, >= H] view (rows may lie apart) of logits, one per head, whose
    sigmoid multiplies the head."""
    T = out.shape[0]
    if a.numel() < T * maps * H * Vd or out.numel() < T * H * Vd:
        raise KernelError("attn_finish: input or output too small")
    ldg = 0
    if gate is not None:
        if gate.dim() != 2 or gate.stride(1) != 1 or gate.shape[1] < H or gate.shape[0] < T or gate.dtype != out.dtype:
            raise KernelError(f"attn_finish: gate {tuple(gate.shape)} {gate.dtype} for {H} heads")
        ldg = gate.stride(0)
    if inv_freq_v is not None and inv_freq_v.numel() != Vd // 2:
        raise KernelError("attn_finish: frequency table does not match the values")
    _check(lib().spite_attn_finish(
        _ptr(a, "a"), dtype_code(a.dtype), _ptr(out, "out"), dtype_code(out.dtype),
        _ptr(positions, "positions", torch.int32, inv_freq_v is None),
        _ptr(inv_freq_v, "inv_freq_v", torch.float32, True), gate.data_ptr() if gate is not None else None, ldg,
        T, H, Vd, int(maps), float(lam), float(eps), float(post), _stream()), "attn_finish")


def token_shift(x, y, w, state, seq_of_token, cu_seqlens, seq_slots, keep=True):
    """y[t] = x[t] + (x[t-1] - x[t]) * w within a request; the first token of an entry takes the
    request's state row for x[t-1], which then receives the entry's last row (``keep``).  x fp32
    [T, d], y [T, d], w fp32 [d], state fp32 [slots, d]."""
    T, d = x.shape
    if y.shape != x.shape or w.numel() != d or state.dim() != 2 or state.shape[1] != d or seq_of_token.numel() < T:
        raise KernelError(f"token_shift: x {tuple(x.shape)}, y {tuple(y.shape)}, state {tuple(state.shape)}")
    _check(lib().spite_token_shift(
        _ptr(x, "x", torch.float32), _ptr(y, "y"), dtype_code(y.dtype), _ptr(w, "w", torch.float32),
        _ptr(state, "state", torch.float32), _ptr(seq_of_token, "seq_of_token", torch.int32),
        _ptr(cu_seqlens, "cu_seqlens", torch.int32), _ptr(seq_slots, "seq_slots", torch.int32), T, d, int(bool(keep)),
        _stream()), "token_shift")


def act_rows(x, act):
    """x = act(x) in place: ``gelu`` (the erf form), ``gelu_tanh`` or ``silu``; fp32 inside."""
    if act not in UNARY_ACTS:
        raise KernelError(f"act_rows: activation {act!r} (known: {sorted(UNARY_ACTS)})")
    _check(lib().spite_act_rows(_ptr(x, "x"), dtype_code(x.dtype), x.numel(), UNARY_ACTS[act], _stream()), "act_rows")


def scale_rows(x, c: float):
    """x *= c in place; x fp32."""
    _check(lib().spite_scale_rows(_ptr(x, "x", torch.float32), x.numel(), float(c), _stream()), "scale_rows")


# -------------------------------------------------------------------------------------------- linear attention
DECAY_FORMS = {"sigmoid_root": 0, "exp_exp": 1}


def channel_decay(z, bias, tau: float = 1.0, form: str = "sigmoid_root"):
    """z[t, c] = sigmoid(z[t, c] + bias[c]) ** (1 / tau) in place (``form`` ``sigmoid_root``), or
    exp(-exp(z[t, c] + bias[c])) (``exp_exp``); z fp32 [T, n], bias fp32 [n] or None."""
    if form not in DECAY_FORMS:
        raise KernelError(f"channel_decay: form {form!r} (known: {sorted(DECAY_FORMS)})")
    T, n = z.shape
    if bias is not None and bias.numel() != n:
        raise KernelError(f"channel_decay: bias of {bias.numel()} for rows of {n}")
    if not tau > 0:
        raise KernelError(f"channel_decay: tau = {tau}")
    _check(lib().spite_channel_decay(_ptr(z, "z", torch.float32), _ptr(bias, "bias", torch.float32, True), T, n,
                                     1.0 / float(tau), DECAY_FORMS[form], _stream()), "channel_decay")


def _rows_view(t, name, width, T):
    """Pointer and row stride of a [T, >= width] view whose rows may lie apart."""
    if t.dim() != 2 or t.stride(1) != 1 or t.shape[0] < T or t.shape[1] < width or not t.is_cuda:
        raise KernelError(f"{name}: {tuple(t.shape)} with strides {t.stride()} for {T} rows of {width}")
    return t.data_ptr(), t.stride(0)


def linear_attn_scan(q, k, v, out, state, cu_seqlens, seq_slots, n_seqs, H, D, V, *, decay=None, head_decay=None,
                     q_scale=1.0, keep=True, longest=0, qk_heads=None, v_scale=None, bonus=None):
    """The recurrence S = diag(a) S + k v^T, o = S^T q token by token for every entry of the step (see
    linear_attn.hip).  q, k [T, H*D] and v [T, H*V]: views of the run's dtype whose rows may lie apart;
    ``decay`` fp32 [T, H*D] (a number per key channel and token) or ``head_decay`` fp32 [H]; ``state`` fp32
    [slots, H, D, V], read at the entry's slot and, with ``keep``, left as the entry's last token leaves it;
    out fp32 [T, H*V].  ``longest``: the most tokens an entry has, if the caller knows (1 picks the kernel made
    for single tokens; the results are the same bits either way).  ``qk_heads`` < H: q and k have that many heads
    ([T, qk_heads*D]) and head h reads head h // (H / qk_heads) of them.  ``v_scale`` fp32 [T, H]: a factor on a
    head's value row as it enters the state.  ``bonus`` fp32 [H, D] (with ``decay``): the result is read before the
    token enters the state, o = (S + diag(bonus) k v^T)^T q."""
    T = out.shape[0]
    Hq = int(qk_heads or H)
    if H % Hq:
        raise KernelError(f"linear_attn_scan: {H} heads over {Hq} heads of q and k")
    if q.dtype != k.dtype or q.dtype != v.dtype:
        raise KernelError("linear_attn_scan: q, k and v of one dtype")
    pq, ldq = _rows_view(q, "q", Hq * D, T)
    pk, ldk = _rows_view(k, "k", Hq * D, T)
    pv, ldv = _rows_view(v, "v", H * V, T)
    if out.numel() < T * H * V or tuple(state.shape[1:]) != (H, D, V):
        raise KernelError(f"linear_attn_scan: out {tuple(out.shape)}, state {tuple(state.shape)} for H={H} D={D} V={V}")
    if decay is not None and decay.numel() < T * H * D:
        raise KernelError("linear_attn_scan: decay too small")
    if head_decay is not None and head_decay.numel() != H:
        raise KernelError(f"linear_attn_scan: {head_decay.numel()} decays for {H} heads")
    if cu_seqlens.numel() < n_seqs + 1 or seq_slots.numel() < n_seqs:
        raise KernelError("linear_attn_scan: metadata too small")
    if v_scale is not None and v_scale.numel() < T * H:
        raise KernelError("linear_attn_scan: v_scale too small")
    if bonus is not None and (bonus.numel() != H * D or decay is None):
        raise KernelError(f"linear_attn_scan: a bonus of {H} x {D} numbers, with a decay per channel")
    _check(lib().spite_linear_attn_scan(
        pq, pk, pv, ldq, ldk, ldv, dtype_code(q.dtype), _ptr(decay, "decay", torch.float32, True),
        _ptr(head_decay, "head_decay", torch.float32, True), float(q_scale), _ptr(state, "state", torch.float32),
        state.shape[0], _ptr(cu_seqlens, "cu_seqlens", torch.int32), _ptr(seq_slots, "seq_slots", torch.int32), int(n_seqs),
        _ptr(out, "out", torch.float32), H, D, V, int(bool(keep)), int(longest), Hq,
        _ptr(v_scale, "v_scale", torch.float32, True), _ptr(bonus, "bonus", torch.float32, True), _stream()), "linear_attn_scan")


NORM_GATES = {None: 0, "silu": 1, "sigmoid": 2}


def gated_group_norm(o, weight, y, group, eps, gate=None, act=None, gate_first=False, skip=None, skip_weight=None,
                     skip_group=0):
    """y = rmsnorm(o over groups of ``group`` elements) * weight * act(gate).  o fp32 [T, n]; weight fp32
    of ``group`` elements (shared by the groups) or of n; gate a [T, n] view in y's dtype (rows may lie
    apart) with ``act`` silu or sigmoid, or None; y [T, n].  ``gate_first``: y = rmsnorm(o * act(gate)) * weight.
    ``skip`` (a [T, n] view in y's dtype) with ``skip_weight`` fp32 [n / skip_group]: o + skip_weight[head] * skip
    stands for o."""
    T, n = o.shape
    ps, lds = (None, 0)
    if skip is not None:
        if skip.dtype != y.dtype or skip_weight is None or skip_group <= 0 or n % skip_group or skip_weight.numel() != n // skip_group:
            raise KernelError("gated_group_norm: the skip rows have the output's dtype and one weight a head")
        ps, lds = _rows_view(skip, "skip", n, T)
    if act not in NORM_GATES or (act is None) != (gate is None):
        raise KernelError(f"gated_group_norm: gate activation {act!r} (known: silu, sigmoid) with a gate, or neither")
    pg, ldg = (None, 0)
    if gate is not None:
        if gate.dtype != y.dtype:
            raise KernelError("gated_group_norm: the gate has the output's dtype")
        pg, ldg = _rows_view(gate, "gate", n, T)
    if y.numel() < T * n:
        raise KernelError("gated_group_norm: output too small")
    _check(lib().spite_gated_group_norm(_ptr(o, "o", torch.float32), pg, ldg, _ptr(weight, "weight", torch.float32),
                                        weight.numel(), _ptr(y, "y"), dtype_code(y.dtype), T, n, int(group), float(eps),
                                        NORM_GATES[act], int(bool(gate_first)), ps, lds,
                                        _ptr(skip_weight, "skip_weight", torch.float32, True), int(skip_group), _stream()),
           "gated_group_norm")


# -------------------------------------------------------------------------------------------- parts around the stream
def add_tanh_norm_can_project(d: int) -> bool:
    """Whether ``add_tanh_norm`` forms projections of rows of this width (the row stays in LDS, four elements a thread)."""
    return d % 4 == 0 and d * 4 <= 48 * 1024


def add_tanh_norm(h, w, b, alpha, out=None, out32=None, d1=None, d2=None, rows=None, n_rows=None, write_h=True, normed=None,
                  proj=None, proj_out=None):
    """h (fp32 [T,d]) += d1 + d2 + mult * (tanh(an * yn) * wn + bn) with ``normed`` = (yn, wn, bn, an, mult); then
    out[i] (and out32[i]) = tanh(alpha * h[r]) * w + b, r = rows[i] or i.  ``w`` None: out is the stream itself in
    out's dtype.  alpha and an are fp32 tensors of one element.  ``proj`` (fp32 [P, d]) with ``proj_out`` (fp32 [T, P]):
    proj_out[i] = proj . (the normed fp32 row i), formed in the same pass (no gathered rows then)."""
    T, d = h.shape
    n = int(n_rows if n_rows is not None else (rows.numel() if rows is not None else T))
    for name, t in (("d1", d1), ("d2", d2)):
        if t is not None and (t.numel() < T * d or t.dtype != torch.float32):
            raise KernelError(f"add_tanh_norm: increment {name} too small or not fp32")
    if w is not None and (w.numel() != d or b is None or b.numel() != d or alpha is None or alpha.numel() != 1):
        raise KernelError(f"add_tanh_norm: weight, bias of {d} elements and one alpha")
    yn = wn = bn = an = None
    mult = 0.0
    if normed is not None:
        yn, wn, bn, an, mult = normed
        if yn.numel() < T * d or wn.numel() != d or bn.numel() != d or an.numel() != 1:
            raise KernelError("add_tanh_norm: the normed increment's sizes")
    if rows is not None and (write_h or rows.numel() < n):
        raise KernelError("add_tanh_norm: gathered rows do not write the stream")
    for name, t in (("out", out), ("out32", out32)):
        if t is not None and t.numel() < n * d:
            raise KernelError(f"add_tanh_norm: {name} too small")
    f = torch.float32
    if proj is not None:
        if rows is not None or w is None or proj.dim() != 2 or proj.shape[1] != d or proj_out is None or proj_out.numel() < n * proj.shape[0] \
                or not add_tanh_norm_can_project(d):
            raise KernelError(f"add_tanh_norm: products {None if proj is None else tuple(proj.shape)} of rows of {d}")
        _check(lib().spite_add_tanh_norm_proj(
            _ptr(h, "h", f), _ptr(d1, "d1", f, True), _ptr(d2, "d2", f, True), _ptr(yn, "yn", f, True), _ptr(wn, "wn", f, True),
            _ptr(bn, "bn", f, True), _ptr(an, "an", f, True), float(mult), _ptr(w, "w", f), _ptr(b, "b", f), _ptr(alpha, "alpha", f),
            _ptr(out, "out", None, True), dtype_code(out.dtype) if out is not None else F32, _ptr(out32, "out32", f, True), n, d,
            int(bool(write_h)), _ptr(proj, "proj", f), _ptr(proj_out, "proj_out", f), proj.shape[0], _stream()), "add_tanh_norm")
        return
    _check(lib().spite_add_tanh_norm(
        _ptr(h, "h", f), _ptr(d1, "d1", f, True), _ptr(d2, "d2", f, True), _ptr(yn, "yn", f, True), _ptr(wn, "wn", f, True),
        _ptr(bn, "bn", f, True), _ptr(an, "an", f, True), float(mult), _ptr(w, "w", f, True), _ptr(b, "b", f, True),
        _ptr(alpha, "alpha", f, True), _ptr(out, "out", None, True), dtype_code(out.dtype) if out is not None else F32,
        _ptr(out32, "out32", f, True), _ptr(rows, "rows", torch.int32, True), n, d, int(bool(write_h)), _stream()), "add_tanh_norm")


def hash_rows(ids, positions, seq_of_token, cu_seqlens, seq_slots, state, rows, mul_prev, mul_cur, buckets, keep=True):
    """rows[t] = (previous token * mul_prev + token * mul_cur) mod buckets, ``buckets`` itself at position 0.  The
    previous token of an entry's first token is state[slot] (int32 [slots]), which then takes the entry's last token."""
    T = rows.numel()
    if ids.numel() < T or positions.numel() < T or seq_of_token.numel() < T or state.dim() != 1:
        raise KernelError("hash_rows: arrays too small")
    i32 = torch.int32
    _check(lib().spite_hash_rows(_ptr(ids, "ids", i32), _ptr(positions, "positions", i32), _ptr(seq_of_token, "seq_of_token", i32),
                                 _ptr(cu_seqlens, "cu_seqlens", i32), _ptr(seq_slots, "seq_slots", i32), _ptr(state, "state", i32),
                                 _ptr(rows, "rows", i32), T, int(mul_prev), int(mul_cur), int(buckets), int(bool(keep)), _stream()),
           "hash_rows")


def embed_sum(ids, table, rows2, table2, h, scale=1.0):
    """h[t] = table[ids[t]] * scale + table2[rows2[t]] as fp32."""
    T, d = h.shape
    if table.shape[1] != d or table2.shape[1] != d or table.dtype != table2.dtype or ids.numel() < T or rows2.numel() < T:
        raise KernelError("embed_sum: tables of the stream's width and one dtype")
    _check(lib().spite_embed_sum(_ptr(ids, "ids", torch.int32), _ptr(table, "table"), _ptr(rows2, "rows2", torch.int32),
                                 _ptr(table2, "table2"), dtype_code(table.dtype), _ptr(h, "h", torch.float32), T, d,
                                 table.shape[0], table2.shape[0], float(scale), _stream()), "embed_sum")


CONV_ACTS = {None: 0, "silu": 1}


def causal_conv(x, w, y, state, seq_of_token, cu_seqlens, seq_slots, bias=None, act=None, keep=True):
    """y[t, c] = act(bias[c] + sum_j w[j, c] * x[t - taps + 1 + j, c]) within a request; the inputs before an entry's
    first token come from state (fp32 [slots, taps-1, C]), which then holds the request's last taps - 1 inputs.  x and y:
    [T, C] views of one dtype whose rows may lie apart; w fp32 [taps, C], tap by tap (a checkpoint's [C, taps] transposed)."""
    T = y.shape[0]
    taps, C = w.shape
    px, ldx = _rows_view(x, "x", C, T)
    py, ldy = _rows_view(y, "y", C, T)
    if x.dtype != y.dtype or act not in CONV_ACTS or (bias is not None and bias.numel() != C):
        raise KernelError("causal_conv: x and y of one dtype, activation silu or none, a bias per channel")
    if taps > 1 and (state is None or tuple(state.shape[1:]) != (taps - 1, C)):
        raise KernelError(f"causal_conv: state {None if state is None else tuple(state.shape)} for {taps} taps on {C} channels")
    if seq_of_token.numel() < T or cu_seqlens.numel() != seq_slots.numel() + 1:
        raise KernelError("causal_conv: metadata too small, or not one more running count than entries")
    _check(lib().spite_causal_conv(px, ldx, dtype_code(x.dtype), _ptr(w, "w", torch.float32), _ptr(bias, "bias", torch.float32, True),
                                   _ptr(state, "state", torch.float32, True), _ptr(seq_of_token, "seq_of_token", torch.int32),
                                   _ptr(cu_seqlens, "cu_seqlens", torch.int32), _ptr(seq_slots, "seq_slots", torch.int32),
                                   int(seq_slots.numel()), py, ldy, dtype_code(y.dtype), T, C, taps, CONV_ACTS[act], int(bool(keep)),
                                   _stream()), "causal_conv")


def shift_mix(x, mu, state, y, seq_of_token, cu_seqlens, seq_slots, keep=True):
    """y[s, t] = x[t] + (x[t-1] - x[t]) * mu[s] within a request, s over the rows of mu (fp32 [n, d]); the row before
    an entry's first token is state[slot] (fp32 [slots, d]), which then takes the entry's last row.  x [T, d], y [n, T, d]."""
    T, d = x.shape
    n = mu.shape[0]
    if tuple(y.shape) != (n, T, d) or y.dtype != x.dtype or mu.shape[1] != d or tuple(state.shape[1:]) != (d,) or seq_of_token.numel() < T:
        raise KernelError(f"shift_mix: x {tuple(x.shape)}, mu {tuple(mu.shape)}, y {tuple(y.shape)}, state {tuple(state.shape)}")
    _check(lib().spite_shift_mix(_ptr(x, "x"), dtype_code(x.dtype), _ptr(mu, "mu", torch.float32), _ptr(state, "state", torch.float32),
                                 _ptr(y, "y"), _ptr(seq_of_token, "seq_of_token", torch.int32), _ptr(cu_seqlens, "cu_seqlens", torch.int32),
                                 _ptr(seq_slots, "seq_slots", torch.int32), T, d, n, int(bool(keep)), _stream()), "shift_mix")


def step_decay(raw, dt_bias, a_log, dt, decay, H, N):
    """dt[t, h] = softplus(raw[t, h] + dt_bias[h]); decay[t, h*N + n] = exp(-exp(a_log[h]) * dt[t, h]).  raw: a [T, H]
    view whose rows may lie apart; dt fp32 [T, H]; decay fp32 [T, H*N]."""
    T = dt.shape[0]
    pr, ld = _rows_view(raw, "raw", H, T)
    if dt.numel() < T * H or decay.numel() < T * H * N or dt_bias.numel() != H or a_log.numel() != H:
        raise KernelError("step_decay: arrays too small")
    _check(lib().spite_step_decay(pr, ld, dtype_code(raw.dtype), _ptr(dt_bias, "dt_bias", torch.float32), _ptr(a_log, "a_log", torch.float32),
                                  _ptr(dt, "dt", torch.float32), _ptr(decay, "decay", torch.float32), T, H, N, _stream()), "step_decay")


def softcap_rows(x, cap: float):
    """x = cap * tanh(x / cap) in place; x fp32."""
    _check(lib().spite_softcap_rows(_ptr(x, "x", torch.float32), x.numel(), float(cap), _stream()), "softcap_rows")


def axpby_rows(x, y, out, a: float, b: float):
    """out = a * x + b * y; all fp32 of one size (out may be x or y)."""
    if x.numel() != y.numel() or out.numel() != x.numel():
        raise KernelError("axpby_rows: sizes differ")
    f = torch.float32
    _check(lib().spite_axpby_rows(_ptr(x, "x", f), _ptr(y, "y", f), _ptr(out, "out", f), x.numel(), float(a), float(b), _stream()),
           "axpby_rows")


def concat_rows(a, b, out):
    """out[t] = [a[t] | b[t]] in out's dtype; a, b fp32 [T, d], out [T, 2d]."""
    T, d = a.shape
    if tuple(b.shape) != (T, d) or tuple(out.shape) != (T, 2 * d):
        raise KernelError("concat_rows: shapes")
    f = torch.float32
    _check(lib().spite_concat_rows(_ptr(a, "a", f), _ptr(b, "b", f), _ptr(out, "out"), dtype_code(out.dtype), T, d, _stream()), "concat_rows")


def bias_rows(y, v, out):
    """out[t] = y[t] + v; y, out fp32 [T, d], v fp32 [d]."""
    T, d = y.shape
    if v.numel() != d or out.numel() < T * d:
        raise KernelError("bias_rows: shapes")
    f = torch.float32
    _check(lib().spite_bias_rows(_ptr(y, "y", f), _ptr(v, "v", f), _ptr(out, "out", f), T, d, _stream()), "bias_rows")
