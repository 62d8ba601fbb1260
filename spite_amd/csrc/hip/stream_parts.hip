// Parts around the residual stream that are no RMS norm and no attention:
//
//   add_tanh_norm:   residual additions + the "dynamic tanh" norm  y = tanh(alpha x) * w + b  (each element on its own, no statistic of the row),
//                    with one increment that passes such a norm of its own on its way into the stream
//   hash_rows / embed_sum:  a second embedding whose row is a hash of (previous token, token); the previous token
//                    of a request is kept in a state row
//   causal_conv:     a short convolution over time on every channel, with the request's last inputs as state (two
//                    kernels: the results, then the state)
//   shift_mix:       several blends of a row with the request's previous row, one per reader
//   step_decay:      softplus of a step size, and the decay exp(-exp(A) dt) that it gives, spread over channels
//   softcap_rows, axpby_rows, concat_rows, bias_rows: small fp32 row operations
//
// Everything is computed in fp32 whatever the type of the rows; state rows are fp32.
#include "common.h"

// ------------------------------------------------------------------ residual additions + tanh norm
// v = h[r] + d1[r] + d2[r] + mult * (tanh(an * yn[r]) * wn + bn);  h[r] = v (write_h);
// out[i] = tanh(a * v) * w + b  (w null: v itself, the stream in the products' type), out32 likewise in fp32.
// r = rows[i] or i.  alpha values are read from memory (they are tensors of the checkpoint).
template <typename TO>
__global__ __launch_bounds__(256)
void add_tanh_norm_kernel(float* __restrict__ h, const float* __restrict__ d1, const float* __restrict__ d2,
                          const float* __restrict__ yn, const float* __restrict__ wn, const float* __restrict__ bn,
                          const float* __restrict__ alpha_n, float mult,
                          const float* __restrict__ w, const float* __restrict__ b, const float* __restrict__ alpha,
                          TO* __restrict__ out, float* __restrict__ out32, const int* __restrict__ rows,
                          int n_rows, int d, int write_h) {
    const int d4 = d >> 2;
    const size_t n = (size_t)n_rows * d4;
    const float a = alpha ? alpha[0] : 0.f, an = alpha_n ? alpha_n[0] : 0.f;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const size_t ri = i / d4;
        const int c = (int)(i - ri * d4) * 4;
        const size_t r = rows ? (size_t)rows[ri] : ri;
        f32x4 v = *(const f32x4*)(h + r * d + c);
        if (d1) v += *(const f32x4*)(d1 + r * d + c);
        if (d2) v += *(const f32x4*)(d2 + r * d + c);
        if (yn) {
            const f32x4 y = *(const f32x4*)(yn + r * d + c), ww = *(const f32x4*)(wn + c), bb = *(const f32x4*)(bn + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += mult * fmaf(tanhf(an * y[e]), ww[e], bb[e]);
        }
        if (write_h) *(f32x4*)(h + r * d + c) = v;
        f32x4 o = v;
        if (w) {
            const f32x4 ww = *(const f32x4*)(w + c), bb = *(const f32x4*)(b + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = fmaf(tanhf(a * v[e]), ww[e], bb[e]);
        }
        if (out) {
            if constexpr (sizeof(TO) == 2) {
                const bf16x4 o4 = {(bf16)o[0], (bf16)o[1], (bf16)o[2], (bf16)o[3]};
                *(bf16x4*)((bf16*)out + ri * d + c) = o4;
            } else {
                *(f32x4*)((float*)out + ri * d + c) = o;
            }
        }
        if (out32) *(f32x4*)(out32 + ri * d + c) = o;
    }
}

// the same, one element a thread, for rows whose width is no multiple of four
template <typename TO>
__global__ __launch_bounds__(256)
void add_tanh_norm_any_kernel(float* __restrict__ h, const float* __restrict__ d1, const float* __restrict__ d2,
                              const float* __restrict__ yn, const float* __restrict__ wn, const float* __restrict__ bn,
                              const float* __restrict__ alpha_n, float mult,
                              const float* __restrict__ w, const float* __restrict__ b, const float* __restrict__ alpha,
                              TO* __restrict__ out, float* __restrict__ out32, const int* __restrict__ rows,
                              int n_rows, int d, int write_h) {
    const size_t n = (size_t)n_rows * d;
    const float a = alpha ? alpha[0] : 0.f, an = alpha_n ? alpha_n[0] : 0.f;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const size_t ri = i / d;
        const int c = (int)(i - ri * d);
        const size_t r = rows ? (size_t)rows[ri] : ri;
        float v = h[r * d + c];
        if (d1) v += d1[r * d + c];
        if (d2) v += d2[r * d + c];
        if (yn) v += mult * fmaf(tanhf(an * yn[r * d + c]), wn[c], bn[c]);
        if (write_h) h[r * d + c] = v;
        const float o = w ? fmaf(tanhf(a * v), w[c], b[c]) : v;
        if (out) out[ri * d + c] = from_f32<TO>(o);
        if (out32) out32[ri * d + c] = o;
    }
}

// The same with small fp32 products of the normed row formed on the way (router logits): a workgroup a row, the
// normed row kept in LDS, proj_out[i][e] = proj[e] . normed row, a wave a product.  Rows of a multiple of four
// elements that fit the LDS.  Launched with 256 threads a row, or with 1,024 for a step of few rows (single tokens), where
// a row's tanh evaluations are the time.
template <typename TO>
__global__ __launch_bounds__(1024)
void add_tanh_norm_proj_kernel(float* __restrict__ h, const float* __restrict__ d1, const float* __restrict__ d2,
                               const float* __restrict__ yn, const float* __restrict__ wn, const float* __restrict__ bn,
                               const float* __restrict__ alpha_n, float mult,
                               const float* __restrict__ w, const float* __restrict__ b, const float* __restrict__ alpha,
                               TO* __restrict__ out, float* __restrict__ out32, int d, int write_h,
                               const float* __restrict__ proj, float* __restrict__ proj_out, int P) {
    extern __shared__ __attribute__((aligned(16))) float xs[];
    const size_t r = blockIdx.x;
    const float a = alpha[0], an = alpha_n ? alpha_n[0] : 0.f;
    for (int c = threadIdx.x * 4; c < d; c += blockDim.x * 4) {
        f32x4 v = *(const f32x4*)(h + r * d + c);
        if (d1) v += *(const f32x4*)(d1 + r * d + c);
        if (d2) v += *(const f32x4*)(d2 + r * d + c);
        if (yn) {
            const f32x4 y = *(const f32x4*)(yn + r * d + c), ww = *(const f32x4*)(wn + c), bb = *(const f32x4*)(bn + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += mult * fmaf(tanhf(an * y[e]), ww[e], bb[e]);
        }
        if (write_h) *(f32x4*)(h + r * d + c) = v;
        const f32x4 ww = *(const f32x4*)(w + c), bb = *(const f32x4*)(b + c);
        f32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = fmaf(tanhf(a * v[e]), ww[e], bb[e]);
        *(f32x4*)(xs + c) = o;
        if (out) {
            if constexpr (sizeof(TO) == 2) {
                const bf16x4 o4 = {(bf16)o[0], (bf16)o[1], (bf16)o[2], (bf16)o[3]};
                *(bf16x4*)((bf16*)out + r * d + c) = o4;
            } else {
                *(f32x4*)((float*)out + r * d + c) = o;
            }
        }
        if (out32) *(f32x4*)(out32 + r * d + c) = o;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    for (int e = threadIdx.x >> 6; e < P; e += blockDim.x >> 6) {
        const float s = wave_dot_row(proj + (size_t)e * d, xs, d, true, lane);
        if (lane == 0) proj_out[r * P + e] = s;
    }
}

extern "C" int spite_add_tanh_norm_proj(float* h, const float* d1, const float* d2, const float* yn, const float* wn,
                                        const float* bn, const float* alpha_n, float mult, const float* w, const float* b,
                                        const float* alpha, void* out, int out_dtype, float* out32, int n_rows, int d,
                                        int write_h, const float* proj, float* proj_out, int P, hipStream_t st) {
    SP_REQUIRE(n_rows >= 0 && d > 0 && d % 4 == 0 && (size_t)d * 4 <= 48 * 1024 && P > 0, "add_tanh_norm: rows of %d with %d products", d, P);
    SP_REQUIRE(!yn || (wn && bn && alpha_n), "add_tanh_norm: a normed increment needs its weight, bias and alpha");
    SP_REQUIRE(w && b && alpha && proj && proj_out, "add_tanh_norm: the products need the norm and their matrix");
    if (n_rows == 0) return 0;
    auto al = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    SP_REQUIRE(al(h) && al(d1) && al(d2) && al(yn) && al(wn) && al(bn) && al(w) && al(b) && al(out32) && al(proj)
               && (out_dtype == SP_F32 ? al(out) : ((uintptr_t)out & 7) == 0), "add_tanh_norm: rows must start on 16 bytes");
    const size_t sh = (size_t)d * sizeof(float);
    const int threads = n_rows <= 256 && d >= 4096 ? 1024 : (n_rows <= 256 && d >= 2048 ? 512 : 256);
#define SP_TNP(TO) add_tanh_norm_proj_kernel<TO><<<n_rows, threads, sh, st>>>(h, d1, d2, yn, wn, bn, alpha_n, mult, w, b, alpha, (TO*)out, out32, d, write_h, proj, proj_out, P)
    if (out_dtype == SP_F32) SP_TNP(float);
    else if (out_dtype == SP_BF16) SP_TNP(bf16);
    else return sp_fail("add_tanh_norm: unknown dtype %d", out_dtype);
#undef SP_TNP
    SP_LAUNCH_CHECK("add_tanh_norm");
    return 0;
}

extern "C" int spite_add_tanh_norm(float* h, const float* d1, const float* d2, const float* yn, const float* wn,
                                   const float* bn, const float* alpha_n, float mult, const float* w, const float* b,
                                   const float* alpha, void* out, int out_dtype, float* out32, const int* rows,
                                   int n_rows, int d, int write_h, hipStream_t st) {
    SP_REQUIRE(n_rows >= 0 && d > 0, "add_tanh_norm: bad sizes rows=%d d=%d", n_rows, d);
    SP_REQUIRE(!yn || (wn && bn && alpha_n), "add_tanh_norm: a normed increment needs its weight, bias and alpha");
    SP_REQUIRE(!w || (b && alpha), "add_tanh_norm: the norm needs its weight, bias and alpha");
    SP_REQUIRE(!(rows && write_h), "add_tanh_norm: gathered rows do not write the stream");
    if (n_rows == 0) return 0;
    auto al = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    const bool vec = d % 4 == 0 && al(h) && al(d1) && al(d2) && al(yn) && al(wn) && al(bn) && al(w) && al(b) && al(out32)
                     && (out_dtype == SP_F32 ? al(out) : ((uintptr_t)out & 7) == 0);
    const size_t n = (size_t)n_rows * (vec ? d / 4 : d);
    const unsigned grid = (unsigned)((n + 255) / 256 < 65535u * 16 ? (n + 255) / 256 : 65535u * 16);
#define SP_TN(K, TO) K<TO><<<grid, 256, 0, st>>>(h, d1, d2, yn, wn, bn, alpha_n, mult, w, b, alpha, (TO*)out, out32, rows, n_rows, d, write_h)
    if (out_dtype == SP_F32) { if (vec) SP_TN(add_tanh_norm_kernel, float); else SP_TN(add_tanh_norm_any_kernel, float); }
    else if (out_dtype == SP_BF16) { if (vec) SP_TN(add_tanh_norm_kernel, bf16); else SP_TN(add_tanh_norm_any_kernel, bf16); }
    else return sp_fail("add_tanh_norm: unknown dtype %d", out_dtype);
#undef SP_TN
    SP_LAUNCH_CHECK("add_tanh_norm");
    return 0;
}

// ------------------------------------------------------------------ a hashed second embedding
// row[t] = (previous token * mul_prev + token * mul_cur) mod buckets, or `buckets` (the table's last row) for a
// request's first token.  The previous token of an entry's first token is what the request's state row holds; the
// thread that reads it then replaces it with the entry's last token, so every state row is touched by one thread.
__global__ __launch_bounds__(256)
void hash_rows_kernel(const int* __restrict__ ids, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                      const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, int* __restrict__ state,
                      int* __restrict__ rows, int T, long long mul_prev, long long mul_cur, long long buckets, int keep) {
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= T) return;
    const int e = seq_of_token[t];
    const int first = cu_seqlens[e];
    int prev;
    if (t == first) {
        int* sr = state + seq_slots[e];
        prev = *sr;
        if (keep) *sr = ids[cu_seqlens[e + 1] - 1];
    } else {
        prev = ids[t - 1];
    }
    long long r = ((long long)prev * mul_prev + (long long)ids[t] * mul_cur) % buckets;
    if (r < 0) r += buckets;
    rows[t] = positions[t] == 0 ? (int)buckets : (int)r;
}

extern "C" int spite_hash_rows(const int* ids, const int* positions, const int* seq_of_token, const int* cu_seqlens,
                               const int* seq_slots, int* state, int* rows, int T, long long mul_prev, long long mul_cur,
                               long long buckets, int keep, hipStream_t st) {
    SP_REQUIRE(T >= 0 && buckets > 0 && buckets < (1ll << 31), "hash_rows: %lld buckets", buckets);
    if (T == 0) return 0;
    hash_rows_kernel<<<(T + 255) / 256, 256, 0, st>>>(ids, positions, seq_of_token, cu_seqlens, seq_slots, state, rows, T,
                                                      mul_prev, mul_cur, buckets, keep);
    SP_LAUNCH_CHECK("hash_rows");
    return 0;
}

// h[t] = table[ids[t]] * scale + table2[rows2[t]], in fp32.
template <typename T>
__global__ void embed_sum_kernel(const int* __restrict__ ids, const T* __restrict__ table, const int* __restrict__ rows2,
                                 const T* __restrict__ table2, float* __restrict__ h, int d, int vocab, int n2, float scale) {
    const int t = blockIdx.x;
    const int id = ids[t], r2 = rows2[t];
    const bool ok = id >= 0 && id < vocab && r2 >= 0 && r2 < n2;
    const T* a = table + (size_t)(ok ? id : 0) * d;
    const T* b = table2 + (size_t)(ok ? r2 : 0) * d;
    for (int c = threadIdx.x; c < d; c += blockDim.x)
        h[(size_t)t * d + c] = ok ? to_f32<T>(a[c]) * scale + to_f32<T>(b[c]) : 0.f;
}

extern "C" int spite_embed_sum(const int* ids, const void* table, const int* rows2, const void* table2, int dtype, float* h,
                               int T, int d, int vocab, int n2, float scale, hipStream_t st) {
    SP_REQUIRE(T >= 0 && d > 0 && vocab > 0 && n2 > 0, "embed_sum: bad sizes T=%d d=%d vocab=%d rows=%d", T, d, vocab, n2);
    if (T == 0) return 0;
    if (dtype == SP_F32) embed_sum_kernel<float><<<T, 256, 0, st>>>(ids, (const float*)table, rows2, (const float*)table2, h, d, vocab, n2, scale);
    else if (dtype == SP_BF16) embed_sum_kernel<bf16><<<T, 256, 0, st>>>(ids, (const bf16*)table, rows2, (const bf16*)table2, h, d, vocab, n2, scale);
    else return sp_fail("embed_sum: unknown dtype %d", dtype);
    SP_LAUNCH_CHECK("embed_sum");
    return 0;
}

// ------------------------------------------------------------------ short convolution over time
// y[t][c] = bias[c] + sum_j w[j][c] * u[t - taps + 1 + j][c], u before the request's first token being zero, then an
// activation (0 none, 1 silu).  The weights lie tap by tap, [taps][C] (the last tap is the token's own): a wave's loads
// of one tap are consecutive.  The inputs before an entry's first token are the request's state, fp32
// [slots][taps - 1][C], oldest first.  Every thread forms its own results, reading rows of the step where the entry
// has them and the state where it does not; nothing writes the state here.  A second kernel (causal_conv_keep), launched
// behind this one, then leaves the request's last taps - 1 inputs in the state: one thread reads and writes a channel's
// state, so entries of any length are safe.  Sums run over j upwards from the bias, the same for every token wherever
// a request is cut.
#define CONV_MAX_TAPS 32
template <typename TI, typename TO>
__global__ __launch_bounds__(256)
void causal_conv_kernel(const TI* __restrict__ x, int ldx, const float* __restrict__ w, const float* __restrict__ bias,
                        const float* __restrict__ state, const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
                        const int* __restrict__ seq_slots, TO* __restrict__ y, int ldy, int C, int taps, int act) {
    const int t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int e = seq_of_token[t];
    const int first = cu_seqlens[e];
    const int local = t - first, back = taps - 1;
    const float* sr = state + (size_t)seq_slots[e] * back * C + c;
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int r = local - back + j;                    // the input's row, counted from the entry's first
        const float u = r >= 0 ? to_f32<TI>(x[(size_t)(first + r) * ldx + c]) : sr[(size_t)(r + back) * C];
        acc = fmaf(w[(size_t)j * C + c], u, acc);
    }
    y[(size_t)t * ldy + c] = from_f32<TO>(act == 1 ? acc / (1.0f + expf(-acc)) : acc);
}

// bfloat16 rows whose sizes let a thread take eight channels at a time (16-byte loads and stores); the same sums.
#define CONV_VEC_TAPS 8
__global__ __launch_bounds__(256)
void causal_conv_vec_kernel(const bf16* __restrict__ x, int ldx, const float* __restrict__ w, const float* __restrict__ bias,
                            const float* __restrict__ state, const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
                            const int* __restrict__ seq_slots, bf16* __restrict__ y, int ldy, int C, int taps, int act) {
    const int t = blockIdx.x;
    const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
    if (c >= C) return;
    const int e = seq_of_token[t];
    const int first = cu_seqlens[e];
    const int local = t - first, back = taps - 1;
    const float* sr = state + (size_t)seq_slots[e] * back * C + c;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = bias ? bias[c + i] : 0.f;
#pragma unroll
    for (int j = 0; j < CONV_VEC_TAPS; ++j) {
        if (j < taps) {
            const int r = local - back + j;
            float u[8];
            if (r >= 0) {
                const bf16x8 xv = *(const bf16x8*)(x + (size_t)(first + r) * ldx + c);
#pragma unroll
                for (int i = 0; i < 8; ++i) u[i] = (float)xv[i];
            } else {
                const f32x4 s0 = *(const f32x4*)(sr + (size_t)(r + back) * C), s1 = *(const f32x4*)(sr + (size_t)(r + back) * C + 4);
#pragma unroll
                for (int i = 0; i < 4; ++i) { u[i] = s0[i]; u[4 + i] = s1[i]; }
            }
            const f32x4 w0 = *(const f32x4*)(w + (size_t)j * C + c), w1 = *(const f32x4*)(w + (size_t)j * C + c + 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) { acc[i] = fmaf(w0[i], u[i], acc[i]); acc[4 + i] = fmaf(w1[i], u[4 + i], acc[4 + i]); }
        }
    }
    bf16x8 o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (bf16)(act == 1 ? acc[i] / (1.0f + expf(-acc[i])) : acc[i]);
    *(bf16x8*)(y + (size_t)t * ldy + c) = o;
}

// The same for steps of many tokens: a thread takes eight channels of CONV_TILE consecutive tokens, so a row is read once
// for all the taps that use it and the weights once a tile.  A tile whose tokens belong to one entry runs as straight code
// over rows held in registers; a tile across an entry's border falls back to the token-by-token form.  The sums are the
// same in the same order.
#define CONV_TILE 8
template <int TAPS>
__global__ __launch_bounds__(256)
void causal_conv_tile_kernel(const bf16* __restrict__ x, int ldx, const float* __restrict__ w, const float* __restrict__ bias,
                             const float* __restrict__ state, const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
                             const int* __restrict__ seq_slots, bf16* __restrict__ y, int ldy, int C, int act, int T) {
    constexpr int back = TAPS - 1;
    const int t0 = blockIdx.x * CONV_TILE;
    const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
    if (c >= C) return;
    const int n_tok = T - t0 < CONV_TILE ? T - t0 : CONV_TILE;
    float wv[TAPS][8], bv[8];
#pragma unroll
    for (int j = 0; j < TAPS; ++j) {
        const f32x4 w0 = *(const f32x4*)(w + (size_t)j * C + c), w1 = *(const f32x4*)(w + (size_t)j * C + c + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) { wv[j][i] = w0[i]; wv[j][4 + i] = w1[i]; }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) bv[i] = bias ? bias[c + i] : 0.f;
    auto row = [&](int e, int first, int r, float* u) {            // the input's row r, counted from the entry's first
        if (r >= 0) {
            const bf16x8 xv = *(const bf16x8*)(x + (size_t)(first + r) * ldx + c);
#pragma unroll
            for (int i = 0; i < 8; ++i) u[i] = (float)xv[i];
        } else {
            const float* sr = state + ((size_t)seq_slots[e] * back + (r + back)) * C + c;
            const f32x4 s0 = *(const f32x4*)sr, s1 = *(const f32x4*)(sr + 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) { u[i] = s0[i]; u[4 + i] = s1[i]; }
        }
    };
    auto store = [&](int t, const float* acc) {
        bf16x8 o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (bf16)(act == 1 ? acc[i] / (1.0f + expf(-acc[i])) : acc[i]);
        *(bf16x8*)(y + (size_t)t * ldy + c) = o;
    };
    const int e0 = seq_of_token[t0];
    if (e0 == seq_of_token[t0 + n_tok - 1]) {
        const int first = cu_seqlens[e0], local0 = t0 - first;
        float in[CONV_TILE + back][8];
#pragma unroll
        for (int k = 0; k < CONV_TILE + back; ++k) {
            if (k - back < n_tok) row(e0, first, local0 - back + k, in[k]);
            else {
#pragma unroll
                for (int i = 0; i < 8; ++i) in[k][i] = 0.f;
            }
        }
#pragma unroll
        for (int m = 0; m < CONV_TILE; ++m) {
            if (m < n_tok) {
                float acc[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[i] = bv[i];
#pragma unroll
                for (int j = 0; j < TAPS; ++j) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[i] = fmaf(wv[j][i], in[m + j][i], acc[i]);
                }
                store(t0 + m, acc);
            }
        }
        return;
    }
    for (int m = 0; m < n_tok; ++m) {
        const int t = t0 + m, e = seq_of_token[t];
        const int first = cu_seqlens[e], local = t - first;
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = bv[i];
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {
            float u[8];
            row(e, first, local - back + j, u);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = fmaf(wv[j][i], u[i], acc[i]);
        }
        store(t, acc);
    }
}

// The state after the step: the last taps - 1 inputs of (the old state, then the entry's rows).  A thread a (entry, channel).
template <typename TI>
__global__ __launch_bounds__(256)
void causal_conv_keep_kernel(const TI* __restrict__ x, int ldx, float* __restrict__ state, const int* __restrict__ cu_seqlens,
                             const int* __restrict__ seq_slots, int C, int taps) {
    const int e = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int first = cu_seqlens[e], count = cu_seqlens[e + 1] - first, back = taps - 1;
    float* sr = state + (size_t)seq_slots[e] * back * C + c;
    float v[CONV_MAX_TAPS];
#pragma unroll
    for (int k = 0; k < CONV_MAX_TAPS; ++k) {
        v[k] = 0.f;
        if (k < back) {
            const int idx = count + k;                     // among the old state's inputs (idx < back) or the entry's rows
            v[k] = idx < back ? sr[(size_t)idx * C] : to_f32<TI>(x[(size_t)(first + idx - back) * ldx + c]);
        }
    }
#pragma unroll
    for (int k = 0; k < CONV_MAX_TAPS; ++k)
        if (k < back) sr[(size_t)k * C] = v[k];
}

extern "C" int spite_causal_conv(const void* x, int ldx, int x_dtype, const float* w, const float* bias, float* state,
                                 const int* seq_of_token, const int* cu_seqlens, const int* seq_slots, int n_seqs, void* y, int ldy,
                                 int y_dtype, int T, int C, int taps, int act, int keep, hipStream_t st) {
    SP_REQUIRE(T >= 0 && C > 0 && taps >= 1 && taps <= CONV_MAX_TAPS, "causal_conv: %d channels, %d taps (at most %d)", C, taps, CONV_MAX_TAPS);
    SP_REQUIRE(ldx >= C && ldy >= C && (act == 0 || act == 1), "causal_conv: rows shorter than the channels, or activation %d", act);
    SP_REQUIRE(taps == 1 || state, "causal_conv: the request's last inputs need a state");
    SP_REQUIRE(n_seqs >= 0 && n_seqs <= T, "causal_conv: %d entries of %d tokens", n_seqs, T);
    if (T == 0) return 0;
    const dim3 grid(T, (C + 255) / 256);
    SP_REQUIRE(grid.y <= 65535, "causal_conv: too many channels");
    if (x_dtype == SP_BF16 && y_dtype == SP_BF16 && C % 8 == 0 && ldx % 8 == 0 && ldy % 8 == 0 && taps <= CONV_VEC_TAPS
        && ((uintptr_t)x & 15) == 0 && ((uintptr_t)y & 15) == 0 && ((uintptr_t)state & 15) == 0 && ((uintptr_t)w & 15) == 0) {
        const dim3 vgrid(T, (C / 8 + 255) / 256);
        const dim3 tgrid((T + CONV_TILE - 1) / CONV_TILE, (C / 8 + 255) / 256);
#define SP_CT(N) causal_conv_tile_kernel<N><<<tgrid, 256, 0, st>>>((const bf16*)x, ldx, w, bias, state, seq_of_token, cu_seqlens, \
        seq_slots, (bf16*)y, ldy, C, act, T)
        // many tokens a step (portions of prompts): tiles of tokens; few (single tokens): a workgroup a token
        if (T >= 32 * n_seqs && T >= 256 && taps == 4) SP_CT(4);
        else if (T >= 32 * n_seqs && T >= 256 && taps == 3) SP_CT(3);
        else if (T >= 32 * n_seqs && T >= 256 && taps == 2) SP_CT(2);
        else
#undef SP_CT
        causal_conv_vec_kernel<<<vgrid, 256, 0, st>>>((const bf16*)x, ldx, w, bias, state, seq_of_token, cu_seqlens, seq_slots,
                                                      (bf16*)y, ldy, C, taps, act);
    } else if (x_dtype == SP_F32 && y_dtype == SP_F32) {
        causal_conv_kernel<float, float><<<grid, 256, 0, st>>>((const float*)x, ldx, w, bias, state, seq_of_token, cu_seqlens, seq_slots,
                                                               (float*)y, ldy, C, taps, act);
    } else if (x_dtype == SP_BF16 && y_dtype == SP_BF16) {
        causal_conv_kernel<bf16, bf16><<<grid, 256, 0, st>>>((const bf16*)x, ldx, w, bias, state, seq_of_token, cu_seqlens, seq_slots,
                                                             (bf16*)y, ldy, C, taps, act);
    } else return sp_fail("causal_conv: dtypes %d -> %d", x_dtype, y_dtype);
    SP_LAUNCH_CHECK("causal_conv");
    if (keep && taps > 1 && n_seqs > 0) {
        const dim3 kgrid(n_seqs, (C + 255) / 256);
        if (x_dtype == SP_F32) causal_conv_keep_kernel<float><<<kgrid, 256, 0, st>>>((const float*)x, ldx, state, cu_seqlens, seq_slots, C, taps);
        else causal_conv_keep_kernel<bf16><<<kgrid, 256, 0, st>>>((const bf16*)x, ldx, state, cu_seqlens, seq_slots, C, taps);
        SP_LAUNCH_CHECK("causal_conv (state)");
    }
    return 0;
}

// ------------------------------------------------------------------ several blends with the previous row
// y[s][t] = x[t] + (x'[t] - x[t]) * mu[s], s = 0 .. n-1, with x'[t] the row of the token before t in its request (the
// request's state row for an entry's first token; zeros for a request's first token).  The state then takes the
// entry's last row; the thread that reads an element of it is the one that writes it.
template <typename T>
__global__ __launch_bounds__(256)
void shift_mix_kernel(const T* __restrict__ x, const float* __restrict__ mu, float* __restrict__ state, T* __restrict__ y,
                      const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
                      const int* __restrict__ seq_slots, int Tn, int d, int n, int keep) {
    const int t = blockIdx.x;
    const int e = seq_of_token[t];
    const int first = cu_seqlens[e], last = cu_seqlens[e + 1] - 1;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < d; c += gridDim.y * 256) {
        const float a = to_f32<T>(x[(size_t)t * d + c]);
        float before;
        if (t == first) {
            float* sr = state + (size_t)seq_slots[e] * d + c;
            before = *sr;
            if (keep) *sr = to_f32<T>(x[(size_t)last * d + c]);
        } else {
            before = to_f32<T>(x[(size_t)(t - 1) * d + c]);
        }
        for (int s = 0; s < n; ++s)
            y[((size_t)s * Tn + t) * d + c] = from_f32<T>(fmaf(before - a, mu[(size_t)s * d + c], a));
    }
}

// bfloat16 rows of a multiple of eight elements: eight elements a thread, 16-byte loads and stores.
__global__ __launch_bounds__(256)
void shift_mix_vec_kernel(const bf16* __restrict__ x, const float* __restrict__ mu, float* __restrict__ state, bf16* __restrict__ y,
                          const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
                          const int* __restrict__ seq_slots, int Tn, int d, int n, int keep) {
    const int t = blockIdx.x;
    const int e = seq_of_token[t];
    const int first = cu_seqlens[e], last = cu_seqlens[e + 1] - 1;
    for (int c = (blockIdx.y * 256 + threadIdx.x) * 8; c < d; c += gridDim.y * 2048) {
        const bf16x8 av = *(const bf16x8*)(x + (size_t)t * d + c);
        float a[8], before[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) a[i] = (float)av[i];
        if (t == first) {
            float* sr = state + (size_t)seq_slots[e] * d + c;
            const f32x4 s0 = *(const f32x4*)sr, s1 = *(const f32x4*)(sr + 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) { before[i] = s0[i]; before[4 + i] = s1[i]; }
            if (keep) {
                const bf16x8 lv = *(const bf16x8*)(x + (size_t)last * d + c);
                *(f32x4*)sr = f32x4{(float)lv[0], (float)lv[1], (float)lv[2], (float)lv[3]};
                *(f32x4*)(sr + 4) = f32x4{(float)lv[4], (float)lv[5], (float)lv[6], (float)lv[7]};
            }
        } else {
            const bf16x8 bv = *(const bf16x8*)(x + (size_t)(t - 1) * d + c);
#pragma unroll
            for (int i = 0; i < 8; ++i) before[i] = (float)bv[i];
        }
        for (int s = 0; s < n; ++s) {
            const f32x4 m0 = *(const f32x4*)(mu + (size_t)s * d + c), m1 = *(const f32x4*)(mu + (size_t)s * d + c + 4);
            bf16x8 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                o[i] = (bf16)fmaf(before[i] - a[i], m0[i], a[i]);
                o[4 + i] = (bf16)fmaf(before[4 + i] - a[4 + i], m1[i], a[4 + i]);
            }
            *(bf16x8*)(y + ((size_t)s * Tn + t) * d + c) = o;
        }
    }
}

extern "C" int spite_shift_mix(const void* x, int dtype, const float* mu, float* state, void* y, const int* seq_of_token,
                               const int* cu_seqlens, const int* seq_slots, int T, int d, int n, int keep, hipStream_t st) {
    SP_REQUIRE(T >= 0 && d > 0 && n > 0, "shift_mix: bad sizes T=%d d=%d n=%d", T, d, n);
    if (T == 0) return 0;
    auto al = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    if (dtype == SP_BF16 && d % 8 == 0 && al(x) && al(y) && al(mu) && al(state)) {
        const dim3 vgrid(T, (d / 8 + 255) / 256 < 64 ? (d / 8 + 255) / 256 : 64);
        shift_mix_vec_kernel<<<vgrid, 256, 0, st>>>((const bf16*)x, mu, state, (bf16*)y, seq_of_token, cu_seqlens, seq_slots, T, d, n, keep);
        SP_LAUNCH_CHECK("shift_mix");
        return 0;
    }
    const dim3 grid(T, (d + 255) / 256 < 64 ? (d + 255) / 256 : 64);
    if (dtype == SP_F32) shift_mix_kernel<float><<<grid, 256, 0, st>>>((const float*)x, mu, state, (float*)y, seq_of_token, cu_seqlens, seq_slots, T, d, n, keep);
    else if (dtype == SP_BF16) shift_mix_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)x, mu, state, (bf16*)y, seq_of_token, cu_seqlens, seq_slots, T, d, n, keep);
    else return sp_fail("shift_mix: unknown dtype %d", dtype);
    SP_LAUNCH_CHECK("shift_mix");
    return 0;
}

// ------------------------------------------------------------------ step sizes and the decays they give
// dt[t][h] = softplus(raw[t][h] + dt_bias[h]) (no clamp);  decay[t][h*N + n] = exp(-exp(a_log[h]) * dt[t][h]) for
// every n < N: the state-space recurrence's decay per head, spread over the head's state channels for the scan.
template <typename T>
__global__ __launch_bounds__(256)
void step_decay_kernel(const T* __restrict__ raw, int ld, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                       float* __restrict__ dt, float* __restrict__ decay, int Tn, int H, int N) {
    const size_t n = (size_t)Tn * H * N;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const size_t th = i / N;
        const int ch = (int)(i - th * N);
        const size_t t = th / H;
        const int h = (int)(th - t * H);
        const float z = to_f32<T>(raw[t * ld + h]) + dt_bias[h];
        const float step = z > 20.f ? z + log1pf(expf(-z)) : log1pf(expf(z));
        if (ch == 0) dt[th] = step;
        decay[i] = expf(-expf(a_log[h]) * step);
    }
}

// state channels in multiples of four: a thread writes four of a head's channels in one store
template <typename T>
__global__ __launch_bounds__(256)
void step_decay_vec_kernel(const T* __restrict__ raw, int ld, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                           float* __restrict__ dt, float* __restrict__ decay, int Tn, int H, int N) {
    const int n4 = N >> 2;
    const size_t n = (size_t)Tn * H * n4;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const size_t th = i / n4;
        const int ch = (int)(i - th * n4);
        const size_t t = th / H;
        const int h = (int)(th - t * H);
        const float z = to_f32<T>(raw[t * ld + h]) + dt_bias[h];
        const float step = z > 20.f ? z + log1pf(expf(-z)) : log1pf(expf(z));
        if (ch == 0) dt[th] = step;
        const float a = expf(-expf(a_log[h]) * step);
        *(f32x4*)(decay + th * N + ch * 4) = f32x4{a, a, a, a};
    }
}

extern "C" int spite_step_decay(const void* raw, int ld, int dtype, const float* dt_bias, const float* a_log, float* dt,
                                float* decay, int T, int H, int N, hipStream_t st) {
    SP_REQUIRE(T >= 0 && H > 0 && N > 0 && ld >= H, "step_decay: bad sizes T=%d H=%d N=%d ld=%d", T, H, N, ld);
    if (T == 0) return 0;
    if (N % 4 == 0 && ((uintptr_t)decay & 15) == 0) {
        const size_t nv = (size_t)T * H * (N / 4);
        const unsigned vgrid = (unsigned)((nv + 255) / 256 < 65535u * 16 ? (nv + 255) / 256 : 65535u * 16);
        if (dtype == SP_F32) step_decay_vec_kernel<float><<<vgrid, 256, 0, st>>>((const float*)raw, ld, dt_bias, a_log, dt, decay, T, H, N);
        else if (dtype == SP_BF16) step_decay_vec_kernel<bf16><<<vgrid, 256, 0, st>>>((const bf16*)raw, ld, dt_bias, a_log, dt, decay, T, H, N);
        else return sp_fail("step_decay: unknown dtype %d", dtype);
        SP_LAUNCH_CHECK("step_decay");
        return 0;
    }
    const size_t n = (size_t)T * H * N;
    const unsigned grid = (unsigned)((n + 255) / 256 < 65535u * 16 ? (n + 255) / 256 : 65535u * 16);
    if (dtype == SP_F32) step_decay_kernel<float><<<grid, 256, 0, st>>>((const float*)raw, ld, dt_bias, a_log, dt, decay, T, H, N);
    else if (dtype == SP_BF16) step_decay_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)raw, ld, dt_bias, a_log, dt, decay, T, H, N);
    else return sp_fail("step_decay: unknown dtype %d", dtype);
    SP_LAUNCH_CHECK("step_decay");
    return 0;
}

// ------------------------------------------------------------------ small fp32 row operations
// x = cap * tanh(x / cap) in place.
__global__ void softcap_rows_kernel(float* __restrict__ x, size_t n, float cap) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) x[i] = cap * tanhf(x[i] / cap);
}
extern "C" int spite_softcap_rows(float* x, size_t n, float cap, hipStream_t st) {
    SP_REQUIRE(cap > 0.f, "softcap_rows: cap %g", (double)cap);
    if (n == 0) return 0;
    const unsigned grid = (unsigned)((n + 255) / 256 < 65535u ? (n + 255) / 256 : 65535u);
    softcap_rows_kernel<<<grid, 256, 0, st>>>(x, n, cap);
    SP_LAUNCH_CHECK("softcap_rows");
    return 0;
}

// out = a * x + b * y (out may be x or y).
__global__ void axpby_rows_kernel(const float* __restrict__ x, const float* __restrict__ y, float* __restrict__ out, size_t n, float a, float b) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) out[i] = a * x[i] + b * y[i];
}
extern "C" int spite_axpby_rows(const float* x, const float* y, float* out, size_t n, float a, float b, hipStream_t st) {
    if (n == 0) return 0;
    const unsigned grid = (unsigned)((n + 255) / 256 < 65535u ? (n + 255) / 256 : 65535u);
    axpby_rows_kernel<<<grid, 256, 0, st>>>(x, y, out, n, a, b);
    SP_LAUNCH_CHECK("axpby_rows");
    return 0;
}

// out[t] = [a[t] | b[t]] in the products' type: two fp32 streams of width d side by side.
template <typename TO>
__global__ void concat_rows_kernel(const float* __restrict__ a, const float* __restrict__ b, TO* __restrict__ out, int T, int d) {
    const size_t n = (size_t)T * 2 * d;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const size_t t = i / (2 * d);
        const int c = (int)(i - t * 2 * d);
        out[i] = from_f32<TO>(c < d ? a[t * d + c] : b[t * d + c - d]);
    }
}
extern "C" int spite_concat_rows(const float* a, const float* b, void* out, int out_dtype, int T, int d, hipStream_t st) {
    SP_REQUIRE(T >= 0 && d > 0, "concat_rows: bad sizes");
    if (T == 0) return 0;
    const size_t n = (size_t)T * 2 * d;
    const unsigned grid = (unsigned)((n + 255) / 256 < 65535u ? (n + 255) / 256 : 65535u);
    if (out_dtype == SP_F32) concat_rows_kernel<float><<<grid, 256, 0, st>>>(a, b, (float*)out, T, d);
    else if (out_dtype == SP_BF16) concat_rows_kernel<bf16><<<grid, 256, 0, st>>>(a, b, (bf16*)out, T, d);
    else return sp_fail("concat_rows: unknown dtype %d", out_dtype);
    SP_LAUNCH_CHECK("concat_rows");
    return 0;
}

// out[t] = y[t] + v, v a vector of d elements.
__global__ void bias_rows_kernel(const float* __restrict__ y, const float* __restrict__ v, float* __restrict__ out, size_t n, int d) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) out[i] = y[i] + v[i % d];
}
extern "C" int spite_bias_rows(const float* y, const float* v, float* out, int T, int d, hipStream_t st) {
    SP_REQUIRE(T >= 0 && d > 0, "bias_rows: bad sizes");
    const size_t n = (size_t)T * d;
    if (n == 0) return 0;
    const unsigned grid = (unsigned)((n + 255) / 256 < 65535u ? (n + 255) / 256 : 65535u);
    bias_rows_kernel<<<grid, 256, 0, st>>>(y, v, out, n, d);
    SP_LAUNCH_CHECK("bias_rows");
    return 0;
}
