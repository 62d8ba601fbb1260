// Small row-wise kernels: the token shift of a mixer's input, an activation applied in place and a
// constant on fp32 rows (the logits of a model whose output has one).
#include "common.h"

// ------------------------------------------------------------------ token shift
// y[t] = x[t] + (x'[t] - x[t]) * w, with x'[t] the row of the token before t in its request: the
// row t-1 of the step, or, for the first token of an entry, what the request's state row holds
// (zeros for a request's first token: the state is cleared on admission).  The state then takes
// the entry's last row.  The thread that reads an element of the state is the one that writes it,
// after the read, so an entry of any length is safe; x and the state are fp32.
template <typename TO>
__global__ __launch_bounds__(256)
void token_shift_kernel(const float* __restrict__ x, TO* __restrict__ y, const float* __restrict__ w,
                        float* __restrict__ state, const int* __restrict__ seq_of_token,
                        const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, int d, int keep) {
    const int t = blockIdx.x;
    const int e = seq_of_token[t];
    const int first = cu_seqlens[e], last = cu_seqlens[e + 1] - 1;
    const float* xr = x + (size_t)t * d;
    TO* yr = y + (size_t)t * d;
    const int c0 = blockIdx.y * 1024;                      // a workgroup takes 1,024 elements of the row
    const int c1 = c0 + 1024 < d ? c0 + 1024 : d;
    float* sr = t == first ? state + (size_t)seq_slots[e] * d : nullptr;
    const float* xp = t == first ? sr : xr - d;
    const float* xl = x + (size_t)last * d;
    if ((d & 3) == 0) {                                    // (rows of fp32 start on 16 bytes then)
        const int c = c0 + threadIdx.x * 4;
        if (c >= c1) return;
        const f32x4 a = *(const f32x4*)(xr + c), b = *(const f32x4*)(xp + c), ww = *(const f32x4*)(w + c);
        const f32x4 keep4 = (sr && keep) ? *(const f32x4*)(xl + c) : a;
        f32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = a[i] + (b[i] - a[i]) * ww[i];
        if constexpr (sizeof(TO) == 2) {
            bf16x4 o4;
#pragma unroll
            for (int i = 0; i < 4; ++i) o4[i] = (bf16)o[i];
            *(bf16x4*)((bf16*)yr + c) = o4;
        } else {
            *(f32x4*)((float*)yr + c) = o;
        }
        if (sr && keep) *(f32x4*)(sr + c) = keep4;
        return;
    }
    for (int c = c0 + threadIdx.x; c < c1; c += 256) {
        const float a = xr[c];
        yr[c] = from_f32<TO>(a + (xp[c] - a) * w[c]);
        if (sr && keep) sr[c] = xl[c];
    }
}

extern "C" int spite_token_shift(const float* x, void* y, int y_dtype, const float* w, float* state,
                                 const int* seq_of_token, const int* cu_seqlens, const int* seq_slots, int T, int d,
                                 int keep, hipStream_t st) {
    SP_REQUIRE(T >= 0 && d > 0, "token_shift: bad sizes T=%d d=%d", T, d);
    SP_REQUIRE((d + 1023) / 1024 <= 65535, "token_shift: rows of %d", d);
    if (T == 0) return 0;
    const dim3 grid(T, (d + 1023) / 1024);
    auto al = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    SP_REQUIRE((d & 3) != 0 || (al(x) && al(y) && al(w) && al(state)), "token_shift: rows must start on 16 bytes");
    if (y_dtype == SP_F32) token_shift_kernel<float><<<grid, 256, 0, st>>>(x, (float*)y, w, state, seq_of_token, cu_seqlens, seq_slots, d, keep);
    else if (y_dtype == SP_BF16) token_shift_kernel<bf16><<<grid, 256, 0, st>>>(x, (bf16*)y, w, state, seq_of_token, cu_seqlens, seq_slots, d, keep);
    else return sp_fail("token_shift: unknown dtype %d", y_dtype);
    SP_LAUNCH_CHECK("token_shift");
    return 0;
}

// ------------------------------------------------------------------ activation in place
// (the activations: sp_unary in common.h)
template <typename T>
__global__ __launch_bounds__(256)
void act_rows_kernel(T* __restrict__ x, size_t n, int act) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) x[i] = from_f32<T>(sp_unary(to_f32<T>(x[i]), act, false));
}

// eight bfloat16 a thread and step
__global__ __launch_bounds__(256)
void act_rows_bf16x8_kernel(bf16x8* __restrict__ x, size_t n8, int act) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += stride) {
        bf16x8 v = x[i];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (bf16)sp_unary((float)v[e], act, false);
        x[i] = v;
    }
}

extern "C" int spite_act_rows(void* x, int dtype, size_t n, int act, hipStream_t st) {
    SP_REQUIRE(act >= SP_UNARY_GELU && act <= SP_UNARY_TANH, "act_rows: activation %d", act);
    if (n == 0) return 0;
    if (dtype == SP_BF16 && n % 8 == 0 && ((uintptr_t)x & 15) == 0) {
        const size_t n8 = n / 8;
        const int blocks = (int)((n8 + 255) / 256 < 8192 ? (n8 + 255) / 256 : 8192);
        act_rows_bf16x8_kernel<<<blocks, 256, 0, st>>>((bf16x8*)x, n8, act);
    } else {
        const int blocks = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
        if (dtype == SP_F32) act_rows_kernel<float><<<blocks, 256, 0, st>>>((float*)x, n, act);
        else if (dtype == SP_BF16) act_rows_kernel<bf16><<<blocks, 256, 0, st>>>((bf16*)x, n, act);
        else return sp_fail("act_rows: unknown dtype %d", dtype);
    }
    SP_LAUNCH_CHECK("act_rows");
    return 0;
}

// ------------------------------------------------------------------ a constant on fp32 rows, in place
__global__ __launch_bounds__(256)
void scale_rows_kernel(float* __restrict__ x, size_t n, float c) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) x[i] *= c;
}

extern "C" int spite_scale_rows(float* x, size_t n, float c, hipStream_t st) {
    if (n == 0) return 0;
    const int blocks = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    scale_rows_kernel<<<blocks, 256, 0, st>>>(x, n, c);
    SP_LAUNCH_CHECK("scale_rows");
    return 0;
}
