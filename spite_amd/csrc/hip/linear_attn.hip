// Linear attention: a recurrent state per head instead of a cache of keys and values.
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T        (S: D x V per head; a_t decays the rows, one per key channel)
//   o_t = S_t^T q_t
//
// The decay a_t is either a number per key channel that the token decides (`decay` fp32 [T, H*D]) or a
// constant per head (`head_decay` fp32 [H]).  The state lives in fp32 in a row per request slot,
// [slots, H, D, V]; every sum and product of the recurrence is fp32 whatever the type of q, k and v.
//
// Options of the recurrence: `qk_heads` < H: several heads share one q and one k head (head h reads q/k head
// h / (H / qk_heads)); `v_scale` fp32 [T, H]: the token's value row of a head is multiplied by a number in fp32 before it
// enters the state (a step size); `bonus` fp32 [H, D]: the result is read off the state *before* the token enters it, and the
// token's own outer product counts with a weight per key channel instead:
//   o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t,   S_t = diag(a_t) S_(t-1) + k_t v_t^T.
//
// channel_decay:      z -> sigmoid(z + b)^(1/tau) in place, through its logarithm; or z -> exp(-exp(z + b)).
// linear_attn_scan:   the recurrence token by token, in fp32 FMAs, with the tokens' rows staged through LDS in
//                     blocks; its bits do not depend on how a request's tokens are cut into steps.
// gated_group_norm:   y = rmsnorm(o over groups of `group` elements) * w * act(gate), the step between the
//                     recurrence and the output projection.
#include "common.h"
#include <type_traits>

// ------------------------------------------------------------------ decay per channel
// a = sigmoid(z + b)^(1/tau) = exp(log sigmoid(z + b) / tau), log sigmoid(x) = -(max(-x, 0) + log1p(exp(-|x|))).
__global__ __launch_bounds__(256)
void channel_decay_kernel(float* __restrict__ z, const float* __restrict__ bias, size_t n, int width, float inv_tau, int mode) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const float x = z[i] + (bias ? bias[i % width] : 0.f);
        if (mode == 1) { z[i] = expf(-expf(x)); continue; }
        const float ls = -(fmaxf(-x, 0.f) + log1pf(expf(-fabsf(x))));
        z[i] = expf(ls * inv_tau);
    }
}

extern "C" int spite_channel_decay(float* z, const float* bias, int T, int width, float inv_tau, int mode, hipStream_t st) {
    SP_REQUIRE(mode == 0 || mode == 1, "channel_decay: mode %d", mode);
    SP_REQUIRE(T >= 0 && width > 0 && inv_tau > 0.f, "channel_decay: bad sizes T=%d width=%d 1/tau=%g", T, width, (double)inv_tau);
    const size_t n = (size_t)T * width;
    if (n == 0) return 0;
    const int blocks = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    channel_decay_kernel<<<blocks, 256, 0, st>>>(z, bias, n, width, inv_tau, mode);
    SP_LAUNCH_CHECK("channel_decay");
    return 0;
}

// ------------------------------------------------------------------ the recurrence, token by token
// A workgroup of 512 threads takes 16 value columns of one head of one entry of the step and walks the
// entry's tokens in order.  Thread (vc, dg) = (tid / 32, tid % 32) holds, in registers, the state's elements
// S[d][v0 + vc] and S[d][v0 + vc + 8] for D / 32 key channels d (four consecutive ones at 4 dg, and again 128
// further on for the widest heads; two at 2 dg for heads up to 64): 32 lanes read 512 consecutive bytes of a
// token's q, k or decay row from LDS in one wide read without bank conflicts.  The tokens' q, k, decay and value slice go through LDS a block of tokens at a time, two buffers:
// the next block's loads are in flight while this block is computed, and a whole block is one stretch of code:
// only the state's FMA waits for the token before.  The sum over the key channels is a thread's own partial
// sum, four rotations across a row of 16 lanes and one step from the lower row to the upper.  The state tile
// goes through LDS on the way in and out, so that its rows are read and written 64 bytes at a time.
// The walk is bound by latency, not by FMAs or bytes (about a third of a SIMD's issue slots are used): the
// split over 32 lanes a column is there to have more waves to switch between.
// The order of every sum is fixed by D alone: the bits do not depend on how a request's tokens are cut.
#define LA_VC 16        // value columns a workgroup
#define LA_NT 512       // threads a workgroup: 16 columns x 32 lanes
#define LA_DG 32        // lanes that share a column's key channels
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

// The sum over 32 lanes (two rows of 16): the rows' sums, then the lower row's into the upper row (a row's last
// lane to the next row, rows 1 and 3 only).  The upper 16 of the 32 lanes get it.
__device__ __forceinline__ float row32_sum(float x) {
    x = row16_sum(x);
    return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x142, 0xa, 0xf, false));
}

// VEC: q, k, v (bfloat16) and the decay rows start on 16 bytes and D and V are multiples of 8: a fetch is
// 16 bytes.  Otherwise one element.  (Plain loops and no closures: every array below stays in registers.)
#define LA_OWN(r) (PR >= 4 ? ((r) / 4) * 128 + dg * 4 + ((r) % 4) : dg * PR + (r))    // the thread's r-th key channel
// TB: tokens a block: 16 (8 for the widest heads), or 1 for steps of single tokens, whose workgroups then hold
// little LDS and few registers, so that many are resident and their round trips to memory overlap.
template <typename T, int RR, bool CH, bool VEC, int TB, bool PRE>
__global__ __launch_bounds__(LA_NT) __attribute__((amdgpu_waves_per_eu(1, TB == 1 ? 4 : 2)))
void linear_attn_scan_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int ldq, int ldk, int ldv,
                             const float* __restrict__ decay, const float* __restrict__ head_decay, float q_scale,
                             float* __restrict__ state, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots,
                             float* __restrict__ out, int H, int D, int V, int keep, int qk_rep,
                             const float* __restrict__ v_scale, const float* __restrict__ bonus) {
    constexpr int Dp = 16 * RR;                     // key channels, padded
    constexpr int PR = RR / 2;                      // key channels a thread
    constexpr int NQ = CH ? 3 : 2;                  // rows of Dp a token: q, k and, per channel, the decay
    constexpr int per = NQ * Dp + LA_VC;
    // A fetch is one load and no branch around it.  Two lists of fetches a block: A from q, k and the value
    // slice (elements of type T), B from the decay rows (fp32).
    constexpr int WA = VEC ? 8 : 1, WB = VEC ? 4 : 1;               // elements a fetch
    constexpr int CA = (2 * Dp + LA_VC) / WA, CB = CH ? Dp / WB : 1; // fetches a token
    constexpr int UA = (TB * CA + LA_NT - 1) / LA_NT, UB = CH ? (TB * CB + LA_NT - 1) / LA_NT : 0;   // fetches a thread and block
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    constexpr int PV = PR < 4 ? PR : 4;             // key channels an LDS read
    typedef float vec __attribute__((ext_vector_type(PV)));
    using RawA = typename std::conditional<VEC, u32x4, T>::type;
    using RawB = typename std::conditional<VEC, f32x4, float>::type;
    extern __shared__ __attribute__((aligned(16))) float sm[];      // max(2 * TB * per, Dp * 17) floats
    const int e = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * LA_VC;
    const int tid = threadIdx.x, vc = tid / LA_DG, dg = tid % LA_DG;
    const int t_lo = cu_seqlens[e], t_hi = cu_seqlens[e + 1];
    if (t_lo >= t_hi) return;
    const int vcol = v0 + vc;
    const bool vok = vcol < V;
    float* srow = state + ((size_t)seq_slots[e] * H + h) * (size_t)D * V;
    for (int i = tid; i < D * LA_VC; i += LA_NT) {
        const int d = i / LA_VC, c = i % LA_VC;
        sm[d * (LA_VC + 1) + c] = v0 + c < V ? srow[(size_t)d * V + v0 + c] : 0.f;
    }
    __syncthreads();
    float S[PR];
#pragma unroll
    for (int r = 0; r < PR; ++r) {
        const int d = LA_OWN(r);
        S[r] = d < D ? sm[d * (LA_VC + 1) + vc] : 0.f;
    }
    __syncthreads();
    const float hd = CH ? 1.f : head_decay[h];
    const int hq = h / qk_rep, Hq = H / qk_rep;             // the head of q and k that this head reads
    (void)Hq;
    float ub[PRE ? PR : 1];
    if constexpr (PRE) {
#pragma unroll
        for (int r = 0; r < PR; ++r) { const int d = LA_OWN(r); ub[r] = d < D ? bonus[(size_t)h * D + d] : 0.f; }
    }
    RawA na[UA];
    float ns[UA];                                            // the factor on a fetch's elements
    RawB nb[UB > 0 ? UB : 1];
    // Turn `it` computes block `it` from buffer it & 1 while block it + 1 is on its way into the other one;
    // turn -1 only fetches.
    const int n_blocks = (t_hi - t_lo + TB - 1) / TB;
    for (int it = -1; it < n_blocks; ++it) {
        const int t0 = t_lo + it * TB, tn = t0 + TB;                // this block's first token, the next block's
        const bool more = it + 1 < n_blocks;
        if (more) {
#pragma unroll
            for (int u = 0; u < UA; ++u) {
                const int x = tid + u * LA_NT, j = x / CA, e0 = (x % CA) * WA, part = e0 / Dp, d = e0 % Dp;
                // q and k: channel d of the head; the value slice: column v0 + e0 - 2 Dp
                const T* base = part == 0 ? q : part == 1 ? k : v;
                const int ld = part == 0 ? ldq : part == 1 ? ldk : ldv;
                const int col = part < 2 ? hq * D + d : h * V + v0 + (e0 - 2 * Dp);
                const bool ok = j < TB && tn + j < t_hi && (part < 2 ? d < D : v0 + (e0 - 2 * Dp) < V);
                const RawA got = *(const RawA*)(base + (size_t)(ok ? tn + j : t_lo) * ld + (ok ? col : 0));
                na[u] = ok ? got : RawA{};
                ns[u] = part == 0 ? q_scale : (part == 2 && v_scale) ? v_scale[(size_t)(ok ? tn + j : t_lo) * H + h] : 1.f;
            }
#pragma unroll
            for (int u = 0; u < UB; ++u) {
                const int x = tid + u * LA_NT, j = x / CB, d = (x % CB) * WB;
                const bool ok = j < TB && tn + j < t_hi && d < D;
                const RawB got = *(const RawB*)(decay + ((size_t)(ok ? tn + j : t_lo) * H + h) * D + (ok ? d : 0));
                nb[u] = ok ? got : RawB{};
            }
        }
        float accs[TB];
        if (it >= 0) {
            const float* cur = sm + (it & 1) * (TB * per);
            const int n_tok = t_hi - t0 < TB ? t_hi - t0 : TB;
            // a whole block as one stretch of code: only the state's FMA waits for the token before; the reads,
            // the sums across lanes and the stores of different tokens overlap
// token j of the block: the state moves on, and the thread's parts of the two sums over the key channels are kept
#define LA_TOKEN(j)                                                                         \
            {                                                                               \
                const float* row = cur + (j) * per;                                         \
                const float vv = row[NQ * Dp + vc];                                         \
                accs[j] = 0.f;                                                              \
                _Pragma("unroll")                                                           \
                for (int r = 0; r < PR; r += PV) {                                          \
                    const vec q4 = *(const vec*)(row + LA_OWN(r));                          \
                    const vec k4 = *(const vec*)(row + Dp + LA_OWN(r));                     \
                    vec a4;                                                                 \
                    if (CH) a4 = *(const vec*)(row + 2 * Dp + LA_OWN(r));                   \
                    _Pragma("unroll")                                                       \
                    for (int y = 0; y < PV; ++y) {                                          \
                        const float a = CH ? a4[y] : hd;                                    \
                        const float kv = k4[y] * vv;                                        \
                        if (PRE) accs[j] = fmaf(fmaf(ub[r + y], kv, S[r + y]), q4[y], accs[j]); \
                        S[r + y] = fmaf(a, S[r + y], kv);                                   \
                        if (!PRE) accs[j] = fmaf(S[r + y], q4[y], accs[j]);                 \
                    }                                                                       \
                }                                                                           \
            }
            if (n_tok == TB) {
                // no branch between the tokens of a whole block
#pragma unroll
                for (int j = 0; j < TB; ++j) LA_TOKEN(j)
            } else {
#pragma unroll
                for (int j = 0; j < TB; ++j) {
                    accs[j] = 0.f;
                    if (j < n_tok) LA_TOKEN(j)
                }
            }
#undef LA_TOKEN
#pragma unroll
            for (int j = 0; j < TB; ++j) accs[j] = row32_sum(accs[j]);
        }
        if (more) {
            float* buf = sm + ((it + 1) & 1) * (TB * per);
#pragma unroll
            for (int u = 0; u < UA; ++u) {
                const int x = tid + u * LA_NT, j = x / CA, e0 = (x % CA) * WA, part = e0 / Dp;
                if (j < TB && tn + j < t_hi) {
                    float* dst = buf + j * per + (part < 2 ? e0 : e0 + (NQ - 2) * Dp);
                    const float m = ns[u];
                    if constexpr (VEC) {
                        const u32x4 w = na[u];
                        f32x4 lo, hi;
                        lo.x = __builtin_bit_cast(float, w.x << 16) * m, lo.y = __builtin_bit_cast(float, w.x & 0xffff0000u) * m;
                        lo.z = __builtin_bit_cast(float, w.y << 16) * m, lo.w = __builtin_bit_cast(float, w.y & 0xffff0000u) * m;
                        hi.x = __builtin_bit_cast(float, w.z << 16) * m, hi.y = __builtin_bit_cast(float, w.z & 0xffff0000u) * m;
                        hi.z = __builtin_bit_cast(float, w.w << 16) * m, hi.w = __builtin_bit_cast(float, w.w & 0xffff0000u) * m;
                        *(f32x4*)dst = lo;
                        *(f32x4*)(dst + 4) = hi;
                    } else dst[0] = to_f32<T>(na[u]) * m;
                }
            }
#pragma unroll
            for (int u = 0; u < UB; ++u) {
                const int x = tid + u * LA_NT, j = x / CB, d = (x % CB) * WB;
                if (j < TB && tn + j < t_hi) {
                    if constexpr (VEC) *(f32x4*)(buf + j * per + 2 * Dp + d) = nb[u];
                    else buf[j * per + 2 * Dp + d] = nb[u];
                }
            }
        }
        // the block's results leave after the next block's rows are in LDS: waiting for those loads does not wait for these stores
        if (it >= 0 && dg == LA_DG - 1) {
            const int n_tok = t_hi - t0 < TB ? t_hi - t0 : TB;
            float* orow = out + ((size_t)t0 * H + h) * V + vcol;
#pragma unroll
            for (int j = 0; j < TB; ++j) {
                if (j < n_tok && vok) orow[(size_t)j * H * V] = accs[j];
            }
        }
        __syncthreads();
    }
    if (keep) {
#pragma unroll
        for (int r = 0; r < PR; ++r) {
            const int d = LA_OWN(r);
            if (d < D) sm[d * (LA_VC + 1) + vc] = S[r];
        }
        __syncthreads();
        for (int i = tid; i < D * LA_VC; i += LA_NT) {
            const int d = i / LA_VC, c = i % LA_VC;
            if (v0 + c < V) srow[(size_t)d * V + v0 + c] = sm[d * (LA_VC + 1) + c];
        }
    }
}
#undef LA_OWN

struct la_args {
    dim3 grid; hipStream_t st; const void *q, *k, *v; int ldq, ldk, ldv; const float *decay, *head_decay; float q_scale;
    float* state; const int *cu_seqlens, *seq_slots; float* out; int H, D, V, keep, qk_rep; const float *v_scale, *bonus;
};

template <typename T, int RR, bool CH, bool VEC, int TB, bool PRE = false>
static void la_launch(const la_args& a) {
    constexpr int Dp = 16 * RR, per = (CH ? 3 : 2) * Dp + LA_VC;
    constexpr size_t blocks = (size_t)2 * TB * per, tile = (size_t)Dp * (LA_VC + 1);
    constexpr size_t bytes = (blocks > tile ? blocks : tile) * sizeof(float);
    static_assert(bytes <= 64 * 1024, "linear_attn_scan: the token blocks must fit the default LDS limit");
    linear_attn_scan_kernel<T, RR, CH, VEC, TB, PRE><<<a.grid, LA_NT, bytes, a.st>>>(
        (const T*)a.q, (const T*)a.k, (const T*)a.v, a.ldq, a.ldk, a.ldv, a.decay, a.head_decay, a.q_scale, a.state, a.cu_seqlens,
        a.seq_slots, a.out, a.H, a.D, a.V, a.keep, a.qk_rep, a.v_scale, a.bonus);
}

template <typename T, bool VEC, int RR>
static void la_pick_block(const la_args& a, bool single) {
    constexpr int TB = la_block<RR>::tokens;
    const bool ch = a.decay != nullptr;
    if (a.bonus) {                                  // (the caller has made sure that a bonus comes with a decay per channel)
        if (single) la_launch<T, RR, true, VEC, 1, true>(a); else la_launch<T, RR, true, VEC, TB, true>(a);
        return;
    }
    if (single) { if (ch) la_launch<T, RR, true, VEC, 1>(a); else la_launch<T, RR, false, VEC, 1>(a); }
    else { if (ch) la_launch<T, RR, true, VEC, TB>(a); else la_launch<T, RR, false, VEC, TB>(a); }
}

template <typename T, bool VEC>
static void la_pick(const la_args& a, bool single) {
    if (a.D <= 64) la_pick_block<T, VEC, 4>(a, single);
    else if (a.D <= 128) la_pick_block<T, VEC, 8>(a, single);
    else la_pick_block<T, VEC, 16>(a, single);
}

extern "C" int spite_linear_attn_scan(const void* q, const void* k, const void* v, int ldq, int ldk, int ldv, int dtype,
                                      const float* decay, const float* head_decay, float q_scale, float* state, int n_slots,
                                      const int* cu_seqlens, const int* seq_slots, int n_seqs, float* out,
                                      int H, int D, int V, int keep, int longest, int qk_heads, const float* v_scale,
                                      const float* bonus, hipStream_t st) {
    if (qk_heads <= 0) qk_heads = H;
    SP_REQUIRE(H % qk_heads == 0, "linear_attn_scan: %d heads over %d heads of q and k", H, qk_heads);
    SP_REQUIRE(!bonus || decay, "linear_attn_scan: the bonus form goes with a decay per channel");
    SP_REQUIRE(n_seqs >= 0 && H > 0 && D > 0 && V > 0 && n_slots > 0, "linear_attn_scan: bad sizes");
    SP_REQUIRE(D <= LA_MAXD, "linear_attn_scan: %d key channels a head (at most %d)", D, LA_MAXD);
    SP_REQUIRE(ldq >= qk_heads * D && ldk >= qk_heads * D && ldv >= H * V, "linear_attn_scan: rows shorter than the heads");
    SP_REQUIRE((decay != nullptr) != (head_decay != nullptr), "linear_attn_scan: a decay per channel or one per head, one of them");
    SP_REQUIRE(H <= 65535 && (V + LA_VC - 1) / LA_VC <= 65535, "linear_attn_scan: too many heads or value columns");
    SP_REQUIRE(dtype == SP_F32 || dtype == SP_BF16, "linear_attn_scan: unknown dtype %d", dtype);
    if (n_seqs == 0) return 0;
    const la_args a{dim3(n_seqs, H, (V + LA_VC - 1) / LA_VC), st, q, k, v, ldq, ldk, ldv, decay, head_decay, q_scale, state,
                    cu_seqlens, seq_slots, out, H, D, V, keep, H / qk_heads, v_scale, bonus};
    auto on16 = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    const bool vec = dtype == SP_BF16 && D % 8 == 0 && V % 8 == 0 && ldq % 8 == 0 && ldk % 8 == 0 && ldv % 8 == 0
                     && on16(q) && on16(k) && on16(v) && on16(decay);
    const bool single = longest == 1;               // (0: not known)
    if (dtype == SP_F32) la_pick<float, false>(a, single);
    else if (vec) la_pick<bf16, true>(a, single);
    else la_pick<bf16, false>(a, single);
    SP_LAUNCH_CHECK("linear_attn_scan");
    return 0;
}

// ------------------------------------------------------------------ norm over groups, weight, gate
// One wave a (token, group): y[c] = o[c] / sqrt(mean over the group (o^2) + eps) * w[c % n_w] * act(gate[c]),
// act: 1 silu, 2 sigmoid (0: no gate).  o fp32 [T, n]; gate rows `ldg` apart, in y's type.
// `pre_gate`: the gate comes before the norm, y = rmsnorm(o * act(gate)) * w.  `skip` (rows `lds` apart, in y's type)
// with `skip_w` fp32 [n / skip_group]: o[c] + skip_w[c / skip_group] * skip[c] stands for o[c] (a direct path from
// the recurrence's input to its result, one weight a head).
#define GGN_KEEP 8            // values a lane keeps: groups of up to 512 elements are read once
// (the wide form reads its values twice: holding up to 24 of them a thread was measured slower, 40 against 30 us)
struct ggn_extra { const void* skip; int lds; const float* skip_w; int skip_group; int pre_gate; };
template <typename TO>
__device__ __forceinline__ float ggn_value(const float* orow, const TO* gate, int ldg, size_t t, int c0, int c, int act, const ggn_extra& ex) {
    float x = orow[c];
    if (ex.skip) x = fmaf(ex.skip_w[(c0 + c) / ex.skip_group], to_f32<TO>(((const TO*)ex.skip)[t * ex.lds + c0 + c]), x);
    if (ex.pre_gate && act) {
        const float g = to_f32<TO>(gate[t * ldg + c0 + c]);
        const float sg = 1.0f / (1.0f + expf(-g));
        x *= act == 1 ? g * sg : sg;
    }
    return x;
}
template <typename TO>
__global__ __launch_bounds__(256)
void gated_group_norm_kernel(const float* __restrict__ o, const TO* __restrict__ gate, int ldg, const float* __restrict__ w,
                             int n_w, TO* __restrict__ y, int T, int n, int group, float eps, int act, ggn_extra ex) {
    const int lane = threadIdx.x & 63;
    const int groups = n / group;
    const size_t item = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= (size_t)T * groups) return;
    const size_t t = item / groups;
    const int c0 = (int)(item % groups) * group;
    const float* orow = o + t * n + c0;
    float ss = 0.f;
    float kept[GGN_KEEP];                             // a lane's first values stay in registers between the two passes
#pragma unroll
    for (int k = 0; k < GGN_KEEP; ++k) {
        const int c = lane + k * 64;
        kept[k] = c < group ? ggn_value<TO>(orow, gate, ldg, t, c0, c, act, ex) : 0.f;
        ss = fmaf(kept[k], kept[k], ss);
    }
    for (int c = lane + GGN_KEEP * 64; c < group; c += 64) { const float x = ggn_value<TO>(orow, gate, ldg, t, c0, c, act, ex); ss = fmaf(x, x, ss); }
    const float sc = 1.0f / sqrtf(wave_sum(ss) / (float)group + eps);
#pragma unroll
    for (int k = 0; k < GGN_KEEP; ++k) {
        const int c = lane + k * 64;
        if (c >= group) continue;
        float x = kept[k] * sc * w[(c0 + c) % n_w];
        if (act && !ex.pre_gate) {
            const float g = to_f32<TO>(gate[t * ldg + c0 + c]);
            const float sg = 1.0f / (1.0f + expf(-g));
            x *= act == 1 ? g * sg : sg;
        }
        y[t * n + c0 + c] = from_f32<TO>(x);
    }
    for (int c = lane + GGN_KEEP * 64; c < group; c += 64) {
        float x = ggn_value<TO>(orow, gate, ldg, t, c0, c, act, ex) * sc * w[(c0 + c) % n_w];
        if (act && !ex.pre_gate) {
            const float g = to_f32<TO>(gate[t * ldg + c0 + c]);
            const float sg = 1.0f / (1.0f + expf(-g));
            x *= act == 1 ? g * sg : sg;
        }
        y[t * n + c0 + c] = from_f32<TO>(x);
    }
}

// The same for wide groups (the heads normed together): a workgroup a (token, group), the sum of squares across
// its four waves through LDS.
template <typename TO>
__global__ __launch_bounds__(256)
void gated_group_norm_wide_kernel(const float* __restrict__ o, const TO* __restrict__ gate, int ldg, const float* __restrict__ w,
                                  int n_w, TO* __restrict__ y, int n, int group, float eps, int act, ggn_extra ex) {
    __shared__ float part[4];
    const int groups = n / group;
    const size_t t = blockIdx.x / groups;
    const int c0 = (int)(blockIdx.x % groups) * group;
    const float* orow = o + t * n + c0;
    float ss = 0.f;
#pragma unroll 8
    for (int c = threadIdx.x; c < group; c += 256) { const float x = ggn_value<TO>(orow, gate, ldg, t, c0, c, act, ex); ss = fmaf(x, x, ss); }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float sc = 1.0f / sqrtf(((part[0] + part[1]) + (part[2] + part[3])) / (float)group + eps);
    const bool whole = n_w >= n;                      // a weight for every element of the row: no wrapping
#pragma unroll 4
    for (int c = threadIdx.x; c < group; c += 256) {
        float x = ggn_value<TO>(orow, gate, ldg, t, c0, c, act, ex) * sc * w[whole ? c0 + c : (c0 + c) % n_w];
        if (act && !ex.pre_gate) {
            const float g = to_f32<TO>(gate[t * ldg + c0 + c]);
            const float sg = 1.0f / (1.0f + expf(-g));
            x *= act == 1 ? g * sg : sg;
        }
        y[t * n + c0 + c] = from_f32<TO>(x);
    }
}

extern "C" int spite_gated_group_norm(const float* o, const void* gate, int ldg, const float* w, int n_w, void* y, int y_dtype,
                                      int T, int n, int group, float eps, int act, int pre_gate, const void* skip, int lds,
                                      const float* skip_w, int skip_group, hipStream_t st) {
    SP_REQUIRE(!skip || (skip_w && skip_group > 0 && n % skip_group == 0 && lds >= n), "gated_group_norm: skip rows of %d in heads of %d", lds, skip_group);
    const ggn_extra ex{skip, lds, skip_w, skip_group > 0 ? skip_group : 1, pre_gate};
    SP_REQUIRE(T >= 0 && n > 0 && group > 0 && n % group == 0, "gated_group_norm: rows of %d in groups of %d", n, group);
    SP_REQUIRE(n_w > 0 && n % n_w == 0 && (n_w % group == 0 || group % n_w == 0), "gated_group_norm: %d weights for groups of %d", n_w, group);
    SP_REQUIRE(act >= 0 && act <= 2 && (act == 0 || (gate && ldg >= n)), "gated_group_norm: gate");
    SP_REQUIRE(eps > 0.f, "gated_group_norm: the norm needs an eps");
    if (T == 0) return 0;
    const size_t items = (size_t)T * (n / group);
    SP_REQUIRE((items + 3) / 4 < (1u << 31), "gated_group_norm: too many groups");
    if (group >= 512 && items < (1u << 31)) {
        if (y_dtype == SP_F32)
            gated_group_norm_wide_kernel<float><<<(unsigned)items, 256, 0, st>>>(o, (const float*)gate, ldg, w, n_w, (float*)y, n, group, eps, act, ex);
        else if (y_dtype == SP_BF16)
            gated_group_norm_wide_kernel<bf16><<<(unsigned)items, 256, 0, st>>>(o, (const bf16*)gate, ldg, w, n_w, (bf16*)y, n, group, eps, act, ex);
        else return sp_fail("gated_group_norm: unknown dtype %d", y_dtype);
        SP_LAUNCH_CHECK("gated_group_norm");
        return 0;
    }
    const unsigned grid = (unsigned)((items + 3) / 4);
    if (y_dtype == SP_F32)
        gated_group_norm_kernel<float><<<grid, 256, 0, st>>>(o, (const float*)gate, ldg, w, n_w, (float*)y, T, n, group, eps, act, ex);
    else if (y_dtype == SP_BF16)
        gated_group_norm_kernel<bf16><<<grid, 256, 0, st>>>(o, (const bf16*)gate, ldg, w, n_w, (bf16*)y, T, n, group, eps, act, ex);
    else return sp_fail("gated_group_norm: unknown dtype %d", y_dtype);
    SP_LAUNCH_CHECK("gated_group_norm");
    return 0;
}
