// Routers that pick several experts a token, and what surrounds their grouped products.
//
// router_topk: from the router's fp32 logits z [T, E] the `top` experts with the largest choice
// values are taken (the lowest index wins among equals), and each gets a weight.  Two ways of scoring:
//   sigmoid (mode 0): scores s = sigmoid(z); the choice goes by s + bias (bias may be null); an expert's
//     weight is its score s without the bias, divided by the sum of the taken scores if `renorm`;
//   softmax over the taken (mode 1): the choice goes by z + bias; the weights are the softmax of the taken
//     experts' logits z alone (they add up to one; `renorm` has nothing left to do).
// Outputs expert[t*top + j] and weight[t*top + j] in the order of choice:
// "virtual tokens" t*top + j that the expert plan (moe_plan with its fan) sorts by expert.
// moe_combine: out[t] = sum_j weight[t*top + j] * y[t*top + j] (+ extra[t]) in fp32, j in order (no weights: all 1).
// gated_rows: g[t] = gelu_tanh(a[t]) * table[ids[t]][col0 .. col0 + n): a gate on a per-token row
// of a table (a second, small embedding that a layer mixes into the stream).
#include "common.h"

#define TOPK_MAX_PER_LANE 8      // up to 512 experts

__global__ __launch_bounds__(256)
void router_topk_kernel(const float* __restrict__ logits, const float* __restrict__ bias, int* __restrict__ expert,
                        float* __restrict__ weight, int T, int E, int top, int renorm, int mode) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    float s[TOPK_MAX_PER_LANE], c[TOPK_MAX_PER_LANE];
#pragma unroll
    for (int u = 0; u < TOPK_MAX_PER_LANE; ++u) {
        const int e = lane + u * 64;
        s[u] = 0.f; c[u] = -INFINITY;
        if (e < E) {
            const float z = logits[(size_t)t * E + e];
            s[u] = mode == 1 ? z : 1.0f / (1.0f + expf(-z));
            c[u] = s[u] + (bias ? bias[e] : 0.f);
            if (!(c[u] == c[u])) c[u] = -INFINITY;          // a NaN is never chosen before a number
        }
    }
    float sum = 0.f, top_z = -INFINITY;          // mode 1: the sum of exp(z - top_z) over the taken so far
    float mine_w = 0.f; int mine_e = 0;
    for (int j = 0; j < top; ++j) {
        float best = -INFINITY; int be = 0x7fffffff; float bs = 0.f;
#pragma unroll
        for (int u = 0; u < TOPK_MAX_PER_LANE; ++u) {
            const int e = lane + u * 64;
            if (e < E && (c[u] > best || (c[u] == best && e < be))) { best = c[u]; be = e; bs = s[u]; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64); const int oe = __shfl_xor(be, o, 64); const float os = __shfl_xor(bs, o, 64);
            if (ob > best || (ob == best && oe < be)) { best = ob; be = oe; bs = os; }
        }
        // a taken expert leaves the contest: its mark lies below every score
#pragma unroll
        for (int u = 0; u < TOPK_MAX_PER_LANE; ++u) if (lane + u * 64 == be) c[u] = -INFINITY;
        if (mode == 1) {
            const float nz = fmaxf(top_z, bs);
            sum = sum * expf(top_z - nz) + expf(bs - nz);        // (exp(-inf) = 0 at the first)
            top_z = nz;
        } else {
            sum += bs;
        }
        if (lane == j % 64 && j < 64) { mine_w = bs; mine_e = be; }
        if (j >= 64 && lane == 0) { expert[(size_t)t * top + j] = be; weight[(size_t)t * top + j] = bs; }
    }
    if (mode == 1) {
        const float inv = 1.0f / sum;
        if (lane < top && lane < 64) { expert[(size_t)t * top + lane] = mine_e; weight[(size_t)t * top + lane] = expf(mine_w - top_z) * inv; }
        if (top > 64 && lane == 0) for (int j = 64; j < top; ++j) weight[(size_t)t * top + j] = expf(weight[(size_t)t * top + j] - top_z) * inv;
        return;
    }
    const float inv = renorm ? 1.0f / fmaxf(sum, 1e-20f) : 1.0f;
    if (lane < top && lane < 64) { expert[(size_t)t * top + lane] = mine_e; weight[(size_t)t * top + lane] = mine_w * inv; }
    if (renorm && top > 64 && lane == 0) for (int j = 64; j < top; ++j) weight[(size_t)t * top + j] *= inv;
}

extern "C" int spite_router_topk(const float* logits, const float* bias, int* expert, float* weight, int T, int E, int top,
                                 int renorm, int mode, hipStream_t st) {
    SP_REQUIRE(mode == 0 || mode == 1, "router_topk: scoring %d", mode);
    SP_REQUIRE(T >= 0 && E > 0 && E <= 64 * TOPK_MAX_PER_LANE, "router_topk: %d experts, at most %d", E, 64 * TOPK_MAX_PER_LANE);
    SP_REQUIRE(top > 0 && top <= E, "router_topk: %d of %d experts", top, E);
    if (T == 0) return 0;
    router_topk_kernel<<<(T + 3) / 4, 256, 0, st>>>(logits, bias, expert, weight, T, E, top, renorm, mode);
    SP_LAUNCH_CHECK("router_topk");
    return 0;
}

__global__ __launch_bounds__(256)
void moe_combine_kernel(const float* __restrict__ y, const float* __restrict__ weight, const float* __restrict__ extra,
                        float* __restrict__ out, int T, int d, int top) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)T * d) return;
    const size_t t = i / d, c = i - t * d;
    float acc = 0.f;
    for (int j = 0; j < top; ++j) acc = fmaf(weight ? weight[t * top + j] : 1.0f, y[(t * top + j) * d + c], acc);
    if (extra) acc += extra[i];
    out[i] = acc;
}

extern "C" int spite_moe_combine(const float* y, const float* weight, const float* extra, float* out, int T, int d, int top,
                                 hipStream_t st) {
    SP_REQUIRE(T >= 0 && d > 0 && top > 0, "moe_combine: bad sizes T=%d d=%d top=%d", T, d, top);
    if (T == 0) return 0;
    const size_t n = (size_t)T * d;
    SP_REQUIRE((n + 255) / 256 < (1u << 31), "moe_combine: too many elements");
    moe_combine_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(y, weight, extra, out, T, d, top);
    SP_LAUNCH_CHECK("moe_combine");
    return 0;
}

template <typename TA, typename TT>
__global__ __launch_bounds__(256)
void gated_rows_kernel(const TA* __restrict__ a, const int* __restrict__ ids, const TT* __restrict__ table, int ld_table,
                       int col0, TA* __restrict__ g, int T, int n, int fast) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)T * n) return;
    const size_t t = i / n, c = i - t * n;
    const float z = to_f32<TA>(a[i]);
    const float act = 0.5f * z * (1.0f + (fast ? 1.0f - 2.0f / (__expf(2.0f * 0.7978845608028654f * (z + 0.044715f * z * z * z)) + 1.0f)
                                              : tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))));
    g[i] = from_f32<TA>(act * to_f32<TT>(table[(size_t)ids[t] * ld_table + col0 + c]));
}

extern "C" int spite_gated_rows(const void* a, int dtype, const int* ids, const void* table, int table_dtype, int ld_table,
                                int col0, void* g, int T, int n, hipStream_t st) {
    SP_REQUIRE(T >= 0 && n > 0 && col0 >= 0 && col0 + n <= ld_table, "gated_rows: columns %d..%d of %d", col0, col0 + n, ld_table);
    if (T == 0) return 0;
    const unsigned grid = (unsigned)(((size_t)T * n + 255) / 256);
    if (dtype == SP_F32 && table_dtype == SP_F32)
        gated_rows_kernel<float, float><<<grid, 256, 0, st>>>((const float*)a, ids, (const float*)table, ld_table, col0, (float*)g, T, n, 0);
    else if (dtype == SP_BF16 && table_dtype == SP_BF16)
        gated_rows_kernel<bf16, bf16><<<grid, 256, 0, st>>>((const bf16*)a, ids, (const bf16*)table, ld_table, col0, (bf16*)g, T, n, 1);
    else if (dtype == SP_BF16 && table_dtype == SP_F32)
        gated_rows_kernel<bf16, float><<<grid, 256, 0, st>>>((const bf16*)a, ids, (const float*)table, ld_table, col0, (bf16*)g, T, n, 1);
    else return sp_fail("gated_rows: dtypes %d and %d", dtype, table_dtype);
    SP_LAUNCH_CHECK("gated_rows");
    return 0;
}
