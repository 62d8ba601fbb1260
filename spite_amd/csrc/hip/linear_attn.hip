// Linear attention: a recurrent state per head instead of a cache of keys and values.
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T        (S: D x V per head; a_t decays the rows, one per key channel)
//   o_t = S_t^T q_t
//
// The decay a_t is either a number per key channel that the token decides (`decay` fp32 [T, H*D]) or a
// constant per head (`head_decay` fp32 [H]).  The state lives in fp32 in a row per request slot,
// [slots, H, D, V]; every sum and product of the recurrence is fp32 whatever the type of q, k and v.
//
// channel_decay:      z -> sigmoid(z + b)^(1/tau) in place, through its logarithm.
// linear_attn_scan:   the recurrence token by token, in fp32 FMAs, with the tokens' rows staged through LDS in
//                     blocks; its bits do not depend on how a request's tokens are cut into steps.
// gated_group_norm:   y = rmsnorm(o over groups of `group` elements) * w * act(gate), the step between the
//                     recurrence and the output projection.
#include "common.h"

// ------------------------------------------------------------------ decay per channel
// a = sigmoid(z + b)^(1/tau) = exp(log sigmoid(z + b) / tau), log sigmoid(x) = -(max(-x, 0) + log1p(exp(-|x|))).
__global__ __launch_bounds__(256)
void channel_decay_kernel(float* __restrict__ z, const float* __restrict__ bias, size_t n, int width, float inv_tau) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const float x = z[i] + (bias ? bias[i % width] : 0.f);
        const float ls = -(fmaxf(-x, 0.f) + log1pf(expf(-fabsf(x))));
        z[i] = expf(ls * inv_tau);
    }
}

extern "C" int spite_channel_decay(float* z, const float* bias, int T, int width, float inv_tau, hipStream_t st) {
    SP_REQUIRE(T >= 0 && width > 0 && inv_tau > 0.f, "channel_decay: bad sizes T=%d width=%d 1/tau=%g", T, width, (double)inv_tau);
    const size_t n = (size_t)T * width;
    if (n == 0) return 0;
    const int blocks = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    channel_decay_kernel<<<blocks, 256, 0, st>>>(z, bias, n, width, inv_tau);
    SP_LAUNCH_CHECK("channel_decay");
    return 0;
}

// ------------------------------------------------------------------ the recurrence, token by token
// A workgroup of 256 threads takes 16 value columns of one head of one entry of the step and walks the
// entry's tokens in order.  Thread (vc, dg) = (tid / 16, tid % 16) holds the state's elements
// S[dg * RR + r][v0 + vc], r < RR (RR = 4, 8 or 16 for up to 64, 128 or 256 key channels), in registers.
// The tokens' q, k, decay and value slice go through LDS a block of LA_TB tokens at a time, two buffers:
// the next block's loads are in flight while this block is computed, so a token costs its FMAs, a few
// wide LDS reads and four steps across the thread's 16 neighbours, and one barrier a block.  The
// dependent chain from token to token is the one FMA of the state.  The state tile goes through LDS on
// the way in and out, so that its rows are read and written 64 bytes at a time.
// The order of every sum is fixed by D alone: the bits do not depend on how a request's tokens are cut.
#define LA_VC 16
#define LA_DG 16
#define LA_MAXD 256

template <int RR> struct la_block { static constexpr int tokens = RR == 16 ? 8 : 16; };

// The sum over the 16 lanes of a row, by rotations within the row (no LDS traffic); every lane gets it.
__device__ __forceinline__ float row16_sum(float x) {
#define LA_ROR(n) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 | (n), 0xf, 0xf, false))
    x += LA_ROR(8);
    x += LA_ROR(4);
    x += LA_ROR(2);
    x += LA_ROR(1);
#undef LA_ROR
    return x;
}

// VEC: q, k, v (bfloat16) and the decay rows start on 16 bytes and D and V are multiples of 8: a thread
// fetches eight elements at a time.  Otherwise one element at a time.
template <typename T, int RR, bool CH, bool VEC>
__global__ __launch_bounds__(256)
void linear_attn_scan_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int ldq, int ldk, int ldv,
                             const float* __restrict__ decay, const float* __restrict__ head_decay, float q_scale,
                             float* __restrict__ state, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots,
                             float* __restrict__ out, int H, int D, int V, int keep) {
    constexpr int Dp = LA_DG * RR;                  // key channels, padded
    constexpr int NQ = CH ? 3 : 2;                  // rows of Dp a token: q, k and, per channel, the decay
    constexpr int per = NQ * Dp + LA_VC;
    constexpr int TB = la_block<RR>::tokens;
    constexpr int W = VEC ? 8 : 1;                  // elements a fetch
    constexpr int CPT = per / W;                    // fetches a token
    constexpr int U = (TB * CPT + 255) / 256;       // fetches a thread and block
    extern __shared__ __attribute__((aligned(16))) float sm[];      // max(2 * TB * per, Dp * 17) floats
    const int e = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * LA_VC;
    const int tid = threadIdx.x, vc = tid / LA_DG, dg = tid % LA_DG;
    const int t_lo = cu_seqlens[e], t_hi = cu_seqlens[e + 1];
    if (t_lo >= t_hi) return;
    const int vcol = v0 + vc;
    const bool vok = vcol < V;
    float* srow = state + ((size_t)seq_slots[e] * H + h) * (size_t)D * V;
    for (int i = tid; i < D * LA_VC; i += 256) {
        const int d = i / LA_VC, c = i % LA_VC;
        sm[d * (LA_VC + 1) + c] = v0 + c < V ? srow[(size_t)d * V + v0 + c] : 0.f;
    }
    __syncthreads();
    float S[RR];
#pragma unroll
    for (int r = 0; r < RR; ++r) {
        const int d = dg * RR + r;
        S[r] = d < D ? sm[d * (LA_VC + 1) + vc] : 0.f;
    }
    __syncthreads();
    const float hd = CH ? 1.f : head_decay[h];
    // elements [W i, W i + W) of a token's row in LDS: [q | k | decay | v slice], each of the first padded with zeros
    auto fetch = [&](int t, int i, float* dst) {
        const int part = (i * W) / Dp, d = (i * W) % Dp;
        if constexpr (VEC) {
#pragma unroll
            for (int x = 0; x < 8; ++x) dst[x] = 0.f;
            if (part < NQ) {
                if (d >= D) return;
                if (part == 2) {
                    const float4* src = (const float4*)(decay + ((size_t)t * H + h) * D + d);
                    const float4 a = src[0], b = src[1];
                    dst[0] = a.x, dst[1] = a.y, dst[2] = a.z, dst[3] = a.w, dst[4] = b.x, dst[5] = b.y, dst[6] = b.z, dst[7] = b.w;
                    return;
                }
                const uint4 raw = *(const uint4*)(part == 0 ? (const void*)(q + (size_t)t * ldq + h * D + d) : (const void*)(k + (size_t)t * ldk + h * D + d));
                const unsigned wds[4] = {raw.x, raw.y, raw.z, raw.w};
                const float m = part == 0 ? q_scale : 1.f;
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    dst[2 * x] = __builtin_bit_cast(float, wds[x] << 16) * m;
                    dst[2 * x + 1] = __builtin_bit_cast(float, wds[x] & 0xffff0000u) * m;
                }
                return;
            }
            const int c = v0 + (i * W - NQ * Dp);
            if (c >= V) return;
            const uint4 raw = *(const uint4*)(v + (size_t)t * ldv + h * V + c);
            const unsigned wds[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                dst[2 * x] = __builtin_bit_cast(float, wds[x] << 16);
                dst[2 * x + 1] = __builtin_bit_cast(float, wds[x] & 0xffff0000u);
            }
        } else {
            if (part < NQ) {
                if (d >= D) dst[0] = 0.f;
                else if (part == 0) dst[0] = to_f32<T>(q[(size_t)t * ldq + h * D + d]) * q_scale;
                else if (part == 1) dst[0] = to_f32<T>(k[(size_t)t * ldk + h * D + d]);
                else dst[0] = decay[((size_t)t * H + h) * D + d];
                return;
            }
            const int c = v0 + (i - NQ * Dp);
            dst[0] = c < V ? to_f32<T>(v[(size_t)t * ldv + h * V + c]) : 0.f;
        }
    };
    float nx[U][W];
    auto load = [&](int t0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int x = tid + u * 256, j = x / CPT, i = x % CPT;
            if (j < TB && t0 + j < t_hi) fetch(t0 + j, i, nx[u]);
        }
    };
    auto put = [&](float* buf, int t0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int x = tid + u * 256, j = x / CPT, i = x % CPT;
            if (j < TB && t0 + j < t_hi) {
                float* dst = buf + j * per + i * W;
                if constexpr (VEC) {
                    *(float4*)dst = make_float4(nx[u][0], nx[u][1], nx[u][2], nx[u][3]);
                    *(float4*)(dst + 4) = make_float4(nx[u][4], nx[u][5], nx[u][6], nx[u][7]);
                } else dst[0] = nx[u][0];
            }
        }
    };
    load(t_lo);
    put(sm, t_lo);
    __syncthreads();
    int b = 0;
    for (int t0 = t_lo; t0 < t_hi; t0 += TB, b ^= 1) {
        const float* cur = sm + b * (TB * per);
        if (t0 + TB < t_hi) load(t0 + TB);
        const int nb = t_hi - t0 < TB ? t_hi - t0 : TB;
        float* orow = out + ((size_t)t0 * H + h) * V + vcol;
        // one token: the state moves on, and the thread's part of the sum over the key channels comes back
        auto token = [&](int j) -> float {
            const float* row = cur + j * per;
            const float vv = row[NQ * Dp + vc];
            float qv[RR], kv[RR], av[RR];
#pragma unroll
            for (int r = 0; r < RR; r += 4) {
                const float4 q4 = *(const float4*)(row + dg * RR + r);
                const float4 k4 = *(const float4*)(row + Dp + dg * RR + r);
                qv[r] = q4.x, qv[r + 1] = q4.y, qv[r + 2] = q4.z, qv[r + 3] = q4.w;
                kv[r] = k4.x, kv[r + 1] = k4.y, kv[r + 2] = k4.z, kv[r + 3] = k4.w;
                if (CH) {
                    const float4 a4 = *(const float4*)(row + 2 * Dp + dg * RR + r);
                    av[r] = a4.x, av[r + 1] = a4.y, av[r + 2] = a4.z, av[r + 3] = a4.w;
                }
            }
            float acc = 0.f;
#pragma unroll
            for (int r = 0; r < RR; ++r) {
                S[r] = fmaf(CH ? av[r] : hd, S[r], kv[r] * vv);
                acc = fmaf(S[r], qv[r], acc);
            }
            return acc;
        };
        if (nb == TB) {
            // a whole block as one stretch of code: only the state's FMA waits for the token before, the reads,
            // the sums across lanes and the stores of different tokens overlap
            float accs[TB];
#pragma unroll
            for (int j = 0; j < TB; ++j) accs[j] = token(j);
#pragma unroll
            for (int j = 0; j < TB; ++j) accs[j] = row16_sum(accs[j]);
            if (dg == 0 && vok) {
#pragma unroll
                for (int j = 0; j < TB; ++j) orow[(size_t)j * H * V] = accs[j];
            }
        } else {
            for (int j = 0; j < nb; ++j) {
                const float acc = row16_sum(token(j));
                if (dg == 0 && vok) orow[(size_t)j * H * V] = acc;
            }
        }
        if (t0 + TB < t_hi) put(sm + (b ^ 1) * (TB * per), t0 + TB);
        __syncthreads();
    }
    if (keep) {
#pragma unroll
        for (int r = 0; r < RR; ++r) {
            const int d = dg * RR + r;
            if (d < D) sm[d * (LA_VC + 1) + vc] = S[r];
        }
        __syncthreads();
        for (int i = tid; i < D * LA_VC; i += 256) {
            const int d = i / LA_VC, c = i % LA_VC;
            if (v0 + c < V) srow[(size_t)d * V + v0 + c] = sm[d * (LA_VC + 1) + c];
        }
    }
}

struct la_args {
    dim3 grid; hipStream_t st; const void *q, *k, *v; int ldq, ldk, ldv; const float *decay, *head_decay; float q_scale;
    float* state; const int *cu_seqlens, *seq_slots; float* out; int H, D, V, keep;
};

template <typename T, int RR, bool CH, bool VEC>
static void la_launch(const la_args& a) {
    constexpr int Dp = LA_DG * RR, per = (CH ? 3 : 2) * Dp + LA_VC, TB = la_block<RR>::tokens;
    constexpr size_t blocks = (size_t)2 * TB * per, tile = (size_t)Dp * (LA_VC + 1);
    constexpr size_t bytes = (blocks > tile ? blocks : tile) * sizeof(float);
    static_assert(bytes <= 64 * 1024, "linear_attn_scan: the token blocks must fit the default LDS limit");
    linear_attn_scan_kernel<T, RR, CH, VEC><<<a.grid, 256, bytes, a.st>>>(
        (const T*)a.q, (const T*)a.k, (const T*)a.v, a.ldq, a.ldk, a.ldv, a.decay, a.head_decay, a.q_scale, a.state, a.cu_seqlens,
        a.seq_slots, a.out, a.H, a.D, a.V, a.keep);
}

template <typename T, bool VEC>
static void la_pick(const la_args& a) {
    const bool ch = a.decay != nullptr;
    if (a.D <= 64) { if (ch) la_launch<T, 4, true, VEC>(a); else la_launch<T, 4, false, VEC>(a); }
    else if (a.D <= 128) { if (ch) la_launch<T, 8, true, VEC>(a); else la_launch<T, 8, false, VEC>(a); }
    else { if (ch) la_launch<T, 16, true, VEC>(a); else la_launch<T, 16, false, VEC>(a); }
}

extern "C" int spite_linear_attn_scan(const void* q, const void* k, const void* v, int ldq, int ldk, int ldv, int dtype,
                                      const float* decay, const float* head_decay, float q_scale, float* state, int n_slots,
                                      const int* cu_seqlens, const int* seq_slots, int n_seqs, float* out,
                                      int H, int D, int V, int keep, hipStream_t st) {
    SP_REQUIRE(n_seqs >= 0 && H > 0 && D > 0 && V > 0 && n_slots > 0, "linear_attn_scan: bad sizes");
    SP_REQUIRE(D <= LA_MAXD, "linear_attn_scan: %d key channels a head (at most %d)", D, LA_MAXD);
    SP_REQUIRE(ldq >= H * D && ldk >= H * D && ldv >= H * V, "linear_attn_scan: rows shorter than the heads");
    SP_REQUIRE((decay != nullptr) != (head_decay != nullptr), "linear_attn_scan: a decay per channel or one per head, one of them");
    SP_REQUIRE(H <= 65535 && (V + LA_VC - 1) / LA_VC <= 65535, "linear_attn_scan: too many heads or value columns");
    SP_REQUIRE(dtype == SP_F32 || dtype == SP_BF16, "linear_attn_scan: unknown dtype %d", dtype);
    if (n_seqs == 0) return 0;
    const la_args a{dim3(n_seqs, H, (V + LA_VC - 1) / LA_VC), st, q, k, v, ldq, ldk, ldv, decay, head_decay, q_scale, state,
                    cu_seqlens, seq_slots, out, H, D, V, keep};
    auto on16 = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    const bool vec = dtype == SP_BF16 && D % 8 == 0 && V % 8 == 0 && ldq % 8 == 0 && ldk % 8 == 0 && ldv % 8 == 0
                     && on16(q) && on16(k) && on16(v) && on16(decay);
    if (dtype == SP_F32) la_pick<float, false>(a);
    else if (vec) la_pick<bf16, true>(a);
    else la_pick<bf16, false>(a);
    SP_LAUNCH_CHECK("linear_attn_scan");
    return 0;
}

// ------------------------------------------------------------------ norm over groups, weight, gate
// One wave a (token, group): y[c] = o[c] / sqrt(mean over the group (o^2) + eps) * w[c % n_w] * act(gate[c]),
// act: 1 silu, 2 sigmoid (0: no gate).  o fp32 [T, n]; gate rows `ldg` apart, in y's type.
template <typename TO>
__global__ __launch_bounds__(256)
void gated_group_norm_kernel(const float* __restrict__ o, const TO* __restrict__ gate, int ldg, const float* __restrict__ w,
                             int n_w, TO* __restrict__ y, int T, int n, int group, float eps, int act) {
    const int lane = threadIdx.x & 63;
    const int groups = n / group;
    const size_t item = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= (size_t)T * groups) return;
    const size_t t = item / groups;
    const int c0 = (int)(item % groups) * group;
    const float* orow = o + t * n + c0;
    float ss = 0.f;
    for (int c = lane; c < group; c += 64) { const float x = orow[c]; ss = fmaf(x, x, ss); }
    const float sc = 1.0f / sqrtf(wave_sum(ss) / (float)group + eps);
    for (int c = lane; c < group; c += 64) {
        float x = orow[c] * sc * w[(c0 + c) % n_w];
        if (act) {
            const float g = to_f32<TO>(gate[t * ldg + c0 + c]);
            const float sg = 1.0f / (1.0f + expf(-g));
            x *= act == 1 ? g * sg : sg;
        }
        y[t * n + c0 + c] = from_f32<TO>(x);
    }
}

extern "C" int spite_gated_group_norm(const float* o, const void* gate, int ldg, const float* w, int n_w, void* y, int y_dtype,
                                      int T, int n, int group, float eps, int act, hipStream_t st) {
    SP_REQUIRE(T >= 0 && n > 0 && group > 0 && n % group == 0, "gated_group_norm: rows of %d in groups of %d", n, group);
    SP_REQUIRE(n_w > 0 && n % n_w == 0 && (n_w % group == 0 || group % n_w == 0), "gated_group_norm: %d weights for groups of %d", n_w, group);
    SP_REQUIRE(act >= 0 && act <= 2 && (act == 0 || (gate && ldg >= n)), "gated_group_norm: gate");
    SP_REQUIRE(eps > 0.f, "gated_group_norm: the norm needs an eps");
    if (T == 0) return 0;
    const size_t items = (size_t)T * (n / group);
    SP_REQUIRE((items + 3) / 4 < (1u << 31), "gated_group_norm: too many groups");
    const unsigned grid = (unsigned)((items + 3) / 4);
    if (y_dtype == SP_F32)
        gated_group_norm_kernel<float><<<grid, 256, 0, st>>>(o, (const float*)gate, ldg, w, n_w, (float*)y, T, n, group, eps, act);
    else if (y_dtype == SP_BF16)
        gated_group_norm_kernel<bf16><<<grid, 256, 0, st>>>(o, (const bf16*)gate, ldg, w, n_w, (bf16*)y, T, n, group, eps, act);
    else return sp_fail("gated_group_norm: unknown dtype %d", y_dtype);
    SP_LAUNCH_CHECK("gated_group_norm");
    return 0;
}
