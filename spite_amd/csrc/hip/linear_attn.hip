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
// linear_attn_scan:   the recurrence token by token: the plain form, whose bits do not depend on how a
//                     request's tokens are cut into steps.
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
// S[dg + 16 r][v0 + vc], r < ceil(D / 16), in registers.  A token's q, k and decay go through LDS (two
// buffers: the next token's are on their way while this one is computed, one barrier a token); the
// sum over the key channels is a thread's own partial sum and four steps across its 16 neighbours.
// The order of every sum is fixed by D alone.
#define LA_VC 16
#define LA_DG 16
#define LA_MAXR 16       // key channels up to 256

template <typename T>
__global__ __launch_bounds__(256)
void linear_attn_scan_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int ldq, int ldk, int ldv,
                             const float* __restrict__ decay, const float* __restrict__ head_decay, float q_scale,
                             float* __restrict__ state, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots,
                             float* __restrict__ out, int H, int D, int V, int keep) {
    extern __shared__ float sm[];                   // [2][3 * D + LA_VC]
    const int e = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * LA_VC;
    const int tid = threadIdx.x, vc = tid / LA_DG, dg = tid % LA_DG;
    const int t_lo = cu_seqlens[e], t_hi = cu_seqlens[e + 1];
    if (t_lo >= t_hi) return;
    const int R = (D + LA_DG - 1) / LA_DG;
    const int vcol = v0 + vc;
    const bool vok = vcol < V;
    float* srow = state + ((size_t)seq_slots[e] * H + h) * (size_t)D * V;
    float S[LA_MAXR];
#pragma unroll
    for (int r = 0; r < LA_MAXR; ++r) {
        const int d = dg + r * LA_DG;
        S[r] = (r < R && d < D && vok) ? srow[(size_t)d * V + vcol] : 0.f;
    }
    const int per = 3 * D + LA_VC;
    const float hd = head_decay ? head_decay[h] : 1.f;
    // what a thread fetches for a token: element i of [q | k | decay | v slice]
    auto fetch = [&](int t, int i) -> float {
        if (i < D) return to_f32<T>(q[(size_t)t * ldq + h * D + i]) * q_scale;
        if (i < 2 * D) return to_f32<T>(k[(size_t)t * ldk + h * D + (i - D)]);
        if (i < 3 * D) return decay ? decay[((size_t)t * H + h) * D + (i - 2 * D)] : hd;
        const int c = v0 + (i - 3 * D);
        return c < V ? to_f32<T>(v[(size_t)t * ldv + h * V + c]) : 0.f;
    };
    // up to four elements a thread (3 * 256 + 16 <= 4 * 256)
    float nx[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) { const int i = tid + u * 256; nx[u] = i < per ? fetch(t_lo, i) : 0.f; }
#pragma unroll
    for (int u = 0; u < 4; ++u) { const int i = tid + u * 256; if (i < per) sm[i] = nx[u]; }
    __syncthreads();
    for (int t = t_lo; t < t_hi; ++t) {
        const float* cur = sm + ((t - t_lo) & 1) * per;
        float* nxt = sm + (((t - t_lo) & 1) ^ 1) * per;
        if (t + 1 < t_hi) {
#pragma unroll
            for (int u = 0; u < 4; ++u) { const int i = tid + u * 256; nx[u] = i < per ? fetch(t + 1, i) : 0.f; }
        }
        const float vv = cur[3 * D + vc];
        float acc = 0.f;
#pragma unroll
        for (int r = 0; r < LA_MAXR; ++r) {
            const int d = dg + r * LA_DG;
            if (r < R && d < D) {
                S[r] = fmaf(cur[2 * D + d], S[r], cur[D + d] * vv);
                acc = fmaf(S[r], cur[d], acc);
            }
        }
        acc += __shfl_xor(acc, 1, 64);
        acc += __shfl_xor(acc, 2, 64);
        acc += __shfl_xor(acc, 4, 64);
        acc += __shfl_xor(acc, 8, 64);
        if (dg == 0 && vok) out[((size_t)t * H + h) * V + vcol] = acc;
        if (t + 1 < t_hi) {
#pragma unroll
            for (int u = 0; u < 4; ++u) { const int i = tid + u * 256; if (i < per) nxt[i] = nx[u]; }
        }
        __syncthreads();
    }
    if (keep) {
#pragma unroll
        for (int r = 0; r < LA_MAXR; ++r) {
            const int d = dg + r * LA_DG;
            if (r < R && d < D && vok) srow[(size_t)d * V + vcol] = S[r];
        }
    }
}

extern "C" int spite_linear_attn_scan(const void* q, const void* k, const void* v, int ldq, int ldk, int ldv, int dtype,
                                      const float* decay, const float* head_decay, float q_scale, float* state, int n_slots,
                                      const int* cu_seqlens, const int* seq_slots, int n_seqs, float* out,
                                      int H, int D, int V, int keep, hipStream_t st) {
    SP_REQUIRE(n_seqs >= 0 && H > 0 && D > 0 && V > 0 && n_slots > 0, "linear_attn_scan: bad sizes");
    SP_REQUIRE(D <= LA_DG * LA_MAXR, "linear_attn_scan: %d key channels a head (at most %d)", D, LA_DG * LA_MAXR);
    SP_REQUIRE(ldq >= H * D && ldk >= H * D && ldv >= H * V, "linear_attn_scan: rows shorter than the heads");
    SP_REQUIRE((decay != nullptr) != (head_decay != nullptr), "linear_attn_scan: a decay per channel or one per head, one of them");
    SP_REQUIRE(H <= 65535 && (V + LA_VC - 1) / LA_VC <= 65535, "linear_attn_scan: too many heads or value columns");
    if (n_seqs == 0) return 0;
    const dim3 grid(n_seqs, H, (V + LA_VC - 1) / LA_VC);
    const size_t sh = (size_t)2 * (3 * D + LA_VC) * sizeof(float);
    if (dtype == SP_F32)
        linear_attn_scan_kernel<float><<<grid, 256, sh, st>>>((const float*)q, (const float*)k, (const float*)v, ldq, ldk, ldv,
            decay, head_decay, q_scale, state, cu_seqlens, seq_slots, out, H, D, V, keep);
    else if (dtype == SP_BF16)
        linear_attn_scan_kernel<bf16><<<grid, 256, sh, st>>>((const bf16*)q, (const bf16*)k, (const bf16*)v, ldq, ldk, ldv,
            decay, head_decay, q_scale, state, cu_seqlens, seq_slots, out, H, D, V, keep);
    else return sp_fail("linear_attn_scan: unknown dtype %d", dtype);
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
