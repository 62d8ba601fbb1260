// Shared declarations of the gfx950 kernel library: element types, error reporting,
// wave-level reductions.  Everything here is written for 64-wide wavefronts.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

typedef __bf16 bf16;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

enum { SP_F32 = 0, SP_BF16 = 1 };
// Which keys a query may read besides the causal rule j <= p: shared with the cache manager.
#define SP_VIS_FN __device__ __host__ __forceinline__
#include "../visibility.h"

#define SP_WAVE 64

// ---- error reporting: every entry point returns 0 or a negative code, and the text of the
// last failure of the calling thread is kept for spite_hip_last_error().
int sp_fail(const char* fmt, ...);
#define SP_REQUIRE(cond, ...) do { if (!(cond)) return sp_fail(__VA_ARGS__); } while (0)
// Compute units of the current device (asked once per device): what tile counts are weighed against.
int sp_cu_count();
// attn_decode.hip: joins the records that split attention leaves (see there).
int sp_attn_combine(const float* part, void* out, int T, int H, int hd, int n_splits, hipStream_t st);
#define SP_LAUNCH_CHECK(name) do { hipError_t e_ = hipGetLastError(); \
    if (e_ != hipSuccess) return sp_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); } while (0)


// ---- layouts of one kv head's part of a cache page.
// Row-major: keys [page_size][hd], values transposed [hd][page_size].
// Operand order (bf16, hd % 32 == 0, page_size % 32 == 0): the MFMA attention kernels' operand
// tiles, each one kilobyte in lane order, so that a wave's load is a run of whole cache lines.
//   keys:   blocks of 32 keys; block b holds two tiles tt of 16 rows, row r of tile tt being the
//           key (r/4)*8 + tt*4 + r%4 of the block, each tile cut into hd/32 chunks cc of 32
//           elements: tile (b, tt, cc) at ((b*2 + tt) * hd/32 + cc) * 512, inside it element
//           8q+e of row r at (q*16 + r)*8 + e.
//   values: block b, 16 head elements dt*16 .. dt*16+15 as rows, the block's 32 keys as k:
//           tile (b, dt) at (b * hd/16 + dt) * 512, inside it key 8q+e of row r at (q*16 + r)*8 + e.
__device__ __forceinline__ size_t sp_k_index(int off, int c, int hd, bool tiled) {
    if (!tiled) return (size_t)off * hd + c;
    const int b = off >> 5, w = off & 31;
    const int r = ((w >> 3) << 2) | (w & 3), tt = (w >> 2) & 1;
    return ((size_t)(b * 2 + tt) * (hd >> 5) + (c >> 5)) * 512 + (size_t)(((((c & 31) >> 3) << 4) + r) << 3) + (c & 7);
}
__device__ __forceinline__ size_t sp_v_index(int c, int off, int hd, int ps, bool tiled) {
    if (!tiled) return (size_t)c * ps + off;
    const int b = off >> 5, w = off & 31;
    return ((size_t)b * (hd >> 4) + (c >> 4)) * 512 + (size_t)((((w >> 3) << 4) + (c & 15)) << 3) + (w & 7);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Which group and which rows the row tile `mt` of a grouped product covers.  Groups are walked
// in order, group e bringing ceil((offsets[e+1] - offsets[e]) / MT) tiles of MT rows.  A wave
// looks at 64 groups at a time (a prefix sum over its lanes), so that hundreds of groups cost a
// few steps; every lane of the wave must call it and gets the same answer.  False: mt lies
// past the last tile.
__device__ __forceinline__ bool sp_find_tile(const int* offsets, int n_groups, int MT, int mt,
                                             int& g, int& row0, int& row_end) {
    const int lane = threadIdx.x & 63;
    int base = 0;
    for (int c = 0; c < n_groups; c += 64) {
        const int e = c + lane;
        int b = 0, en = 0;
        if (e < n_groups) { b = offsets[e]; en = offsets[e + 1]; }
        const int nt = (en - b + MT - 1) / MT;
        int incl = nt;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { const int v = __shfl_up(incl, o, 64); if (lane >= o) incl += v; }
        const int total = __shfl(incl, 63, 64);
        if (mt < base + total) {
            const bool mine = mt >= base + incl - nt && mt < base + incl;
            const int src = __ffsll((unsigned long long)__ballot(mine)) - 1;
            // the same in every lane: say so, to keep them in scalar registers
            g = __builtin_amdgcn_readfirstlane(c + src);
            row0 = __builtin_amdgcn_readfirstlane(__shfl(b, src, 64) + (mt - base - __shfl(incl - nt, src, 64)) * MT);
            row_end = __builtin_amdgcn_readfirstlane(__shfl(en, src, 64));
            return true;
        }
        base += total;
    }
    return false;
}

// Maximum / sum over the four lanes n, n+16, n+32, n+48 of a wave (the four rows of 16 lanes that
// hold one MFMA column), the result in all four.  The row swaps are vector instructions: no
// trip through the LDS crossbar as a shuffle across rows takes.
__device__ __forceinline__ float rows4_max(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float rows4_sum(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Sum over a workgroup of NT threads (NT a multiple of 64, at most 1024); every thread
// gets the result.  `red` is shared scratch of at least NT/64 floats; two barriers.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NT / 64; ++i) t += red[i];
    __syncthreads();
    return t;
}

// ------------------------------------------------------------------ a wave's fp32 dot product
// sum_c w[c] * xs[c] over a row xs in LDS, by one wave: lane l takes the 16-byte groups l, l+64,
// ... and the lanes' sums meet in a butterfly.  Every kernel that forms router logits calls
// this, so a logit has the same bits wherever it is computed; its order of summation depends
// on the width alone.
__device__ __forceinline__ float wave_dot_row(const float* __restrict__ w, const float* xs, int d, bool vec, int lane) {
    float acc = 0.f;
    if (vec) {
        const int nv = d >> 2;
#pragma unroll 10
        for (int c = lane; c < nv; c += 64) {          // independent 16-byte loads, ten in flight
            const f32x4 ww = ((const f32x4*)w)[c];
            const f32x4 xx = ((const f32x4*)xs)[c];
            acc += ww[0] * xx[0] + ww[1] * xx[1] + ww[2] * xx[2] + ww[3] * xx[3];
        }
    } else {
        for (int c = lane; c < d; c += 64) acc += w[c] * xs[c];
    }
    return wave_sum(acc);
}

// The gate's activation in a gated product act(gate) * up: SP_ACT_SILU g * sigmoid(g),
// SP_ACT_GELU_TANH 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))), or SP_ACT_RELU max(g, 0).
// `fast`: the short exponential (the bfloat16 products); the 32-bit path takes the accurate routines.
enum { SP_ACT_NONE = 0, SP_ACT_SILU = 1, SP_ACT_GELU_TANH = 2, SP_ACT_RELU = 3 };
__device__ __forceinline__ float sp_gate_act(float g, int act, bool fast) {
    if (act == SP_ACT_RELU) return fmaxf(g, 0.f);
    if (act == SP_ACT_GELU_TANH) {
        const float z = 0.7978845608028654f * (g + 0.044715f * g * g * g);
        // tanh(z) = 1 - 2 / (exp(2z) + 1): no cancellation where it matters, exact limits at both ends
        const float t = fast ? 1.0f - 2.0f / (__expf(2.0f * z) + 1.0f) : tanhf(z);
        return 0.5f * g * (1.0f + t);
    }
    return g / (1.0f + (fast ? __expf(-g) : expf(-g)));
}

// An activation on its own (no gate): SP_UNARY_GELU 0.5 z (1 + erf(z / sqrt 2)), SP_UNARY_GELU_TANH,
// SP_UNARY_SILU, SP_UNARY_TANH, in fp32.  `fast` (the bfloat16 products' epilogues): the short exponential, and for the
// error function the rational form 1 - (a1 t + ... + a5 t^5) exp(-x^2), t = 1 / (1 + p x), whose error of
// 1.5e-7 is a thousandth of a bfloat16 step; else the accurate routines.  The product kernels take one as
// the epilogue of a plain product: their `glu` argument carries it in the bits above the gate's code
// (glu = unary << 4).
enum { SP_UNARY_GELU = 1, SP_UNARY_GELU_TANH = 2, SP_UNARY_SILU = 3, SP_UNARY_TANH = 4 };
__device__ __forceinline__ float sp_unary(float z, int act, bool fast) {
    if (act == SP_UNARY_GELU) {
        if (!fast) return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f));
        const float x = fabsf(z) * 0.70710678118654752f;
        const float t = __frcp_rn(1.0f + 0.3275911f * x);
        const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
        const float e = 1.0f - poly * __expf(-x * x);              // erf(|z| / sqrt 2)
        return 0.5f * z * (1.0f + copysignf(e, z));
    }
    if (act == SP_UNARY_TANH) return fast ? 1.0f - 2.0f / (__expf(2.0f * z) + 1.0f) : tanhf(z);
    if (act == SP_UNARY_GELU_TANH) return sp_gate_act(z, SP_ACT_GELU_TANH, fast);
    return sp_gate_act(z, SP_ACT_SILU, fast);
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16>(bf16 v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return (bf16)v; }
