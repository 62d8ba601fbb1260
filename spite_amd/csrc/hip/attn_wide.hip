// Attention whose keys and values differ in width and in number of heads, and what stands
// around it: the step between the fused projection and the cache (bias, a norm over the whole
// projection, rotation of a head's leading part, rotation of the values), the plain attention
// kernel, and the step between the attention and the output projection (two score maps of one
// head combined and normed, values turned back, a gate per head).
//
// Heads: HQ query heads and GK key heads of D elements, GV value heads of Vd elements.  Query
// head h reads key head g = h / (HQ / GK) and value head g % GV: with GK = GV this is grouped-query
// attention; with GK = 2 GV the query heads [0, HQ/2) and [HQ/2, HQ) are two score maps over
// the same values (the caller lays the projection's rows out map by map).
//
// Everything the kernels compute between loads and stores is fp32: angles, sines and cosines
// (the accurate routines), sums of squares, scores, softmax, the sums over values.
#include "common.h"

#define WIDE_NT 256
#define QKV_MAX_HPB 16     // heads a workgroup of qkv_prepare, at most

// ------------------------------------------------------------------ projection row -> q, cache
// A workgroup takes `hpb` heads of one token (query heads first, then key heads, then value heads; with
// few tokens a step the heads are dealt to many workgroups, each of which forms the norm's sums over the
// whole q or k part again).  The row holds [HQ*D | GK*D | GV*Vd | ...] (`ld` elements to the next
// row).  x = row + bias; with `wq` / `wk` the q and the k region are each divided by the root mean
// square of the whole region and multiplied by their weights; then the first `rot` elements
// of every q and k head turn by pos * inv_freq[i] in pairs (i, i + rot/2), sine and cosine both
// times `rot_mag` (1: a pure rotation; frequency scalings that stretch the context bring a
// constant above 1 that sharpens the scores of the turning part); with `inv_freq_v` the
// values turn by pos * inv_freq_v[m] in pairs (m, m + Vd/2).  Keys go to [page][GK][offset][Dp],
// values to [page][GV][Vd][offset] (or the operand order of common.h).  Dp >= D is the width that
// queries and keys are stored with: the elements behind D are written as zeros (a head narrower than
// what an attention kernel takes is widened this way; zeros add nothing to a score).
template <typename T>
__global__ __launch_bounds__(WIDE_NT)
void qkv_prepare_kernel(const T* __restrict__ qkv, int ld, const float* __restrict__ bias,
                        const float* __restrict__ wq, const float* __restrict__ wk, float eps,
                        T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
                        const int* __restrict__ positions, const int* __restrict__ slot_map,
                        const float* __restrict__ inv_freq, int rot, float rot_mag, const float* __restrict__ inv_freq_v,
                        int HQ, int GK, int GV, int D, int Vd, int ps, int k_tiled, int v_tiled, int Dp, int hpb,
                        int head_norm, float qt_coef, int qt_every, int v_from_k) {
    extern __shared__ float sm[];
    __shared__ float red[WIDE_NT / 64];
    const int rh = rot >> 1, vh = inv_freq_v ? (Vd >> 1) : 0;
    float* cs = sm;             // [rh]
    float* sn = cs + rh;        // [rh]
    float* csv = sn + rh;       // [vh]
    float* snv = csv + vh;      // [vh]
    const int t = blockIdx.x, tid = threadIdx.x;
    const float pos = (float)positions[t];
    const T* row = qkv + (size_t)t * ld;
    const int Nq = HQ * D, Nk = GK * D;
    for (int i = tid; i < rh; i += WIDE_NT) { float sv, cv; sincosf(pos * inv_freq[i], &sv, &cv); sn[i] = sv * rot_mag; cs[i] = cv * rot_mag; }
    for (int i = tid; i < vh; i += WIDE_NT) sincosf(pos * inv_freq_v[i], &snv[i], &csv[i]);
    const int slot = slot_map ? slot_map[t] : -1;
    // this workgroup's heads [h_lo, h_hi) of the HQ + GK + GV; keys and values only where the token has a cache row
    const int h_lo = blockIdx.y * hpb, h_end = h_lo + hpb;
    const int qk_end = HQ + (slot >= 0 ? GK : 0);
    const int qk_hi = h_end < qk_end ? h_end : qk_end;               // q and k heads [h_lo, qk_hi)
    const int v_lo = (h_lo > HQ + GK ? h_lo : HQ + GK) - (HQ + GK);
    const int v_hi = (h_end < HQ + GK + GV ? h_end : HQ + GK + GV) - (HQ + GK);       // value heads [v_lo, v_hi)
    float scale_q = 1.f, scale_k = 1.f;
    __shared__ float head_sc[QKV_MAX_HPB];
    if (head_norm) {
        // a norm per head: a wave forms the sum of squares of one head of this workgroup at a time
        for (int hh = h_lo + (tid >> 6); hh < qk_hi; hh += WIDE_NT / 64) {
            float s = 0.f;
            for (int c = tid & 63; c < D; c += 64) { const float x = to_f32<T>(row[hh * D + c]) + (bias ? bias[hh * D + c] : 0.f); s += x * x; }
            s = wave_sum(s);
            if ((tid & 63) == 0) head_sc[hh - h_lo] = 1.0f / sqrtf(s / (float)D + eps);
        }
    }
    // the query's temperature: a factor that grows with the logarithm of the position, in steps
    const float q_temp = qt_every > 0 ? 1.0f + qt_coef * logf((float)((positions[t] + 1) / qt_every) + 1.0f) : 1.0f;
    if (!head_norm && wq && h_lo < HQ) {
        float s = 0.f;
        for (int c = tid; c < Nq; c += WIDE_NT) { const float x = to_f32<T>(row[c]) + (bias ? bias[c] : 0.f); s += x * x; }
        scale_q = 1.0f / sqrtf(block_sum<WIDE_NT>(s, red) / (float)Nq + eps);
    }
    if (!head_norm && wk && h_lo < qk_end && h_end > HQ) {
        float s = 0.f;
        for (int c = tid; c < Nk; c += WIDE_NT) { const float x = to_f32<T>(row[Nq + c]) + (bias ? bias[Nq + c] : 0.f); s += x * x; }
        scale_k = 1.0f / sqrtf(block_sum<WIDE_NT>(s, red) / (float)Nk + eps);
    }
    __syncthreads();
    const size_t page = slot >= 0 ? (size_t)(slot / ps) : 0;
    const int off = slot >= 0 ? slot % ps : 0;
    // a head of D elements is rh pairs and D - rot elements that pass through
    const int items = D - rh;
    const int n_qk = (qk_hi > h_lo ? qk_hi - h_lo : 0) * items;
    for (int it = tid; it < n_qk; it += WIDE_NT) {
        const int hh = h_lo + it / items, i = it % items;
        const bool is_q = hh < HQ;
        const int base = hh * D;                       // the q and k regions follow each other in the row
        const float* wn = is_q ? wq : wk;
        const float sc = head_norm ? head_sc[hh - h_lo] : (is_q ? scale_q : scale_k);
        const int wbase = head_norm ? 0 : (is_q ? base : base - Nq);      // a head norm's weights serve every head
        const float qt = is_q ? q_temp : 1.0f;
        auto load = [&](int c) {
            float x = to_f32<T>(row[base + c]) + (bias ? bias[base + c] : 0.f);
            if (wn) x = x * sc * wn[wbase + c];
            return x * qt;
        };
        T* dst = nullptr;
        if (is_q) dst = q_out + ((size_t)t * HQ + hh) * Dp;
        else dst = k_pages + (page * GK + (hh - HQ)) * (size_t)ps * Dp;
        auto store = [&](int c, float v) {
            if (is_q) dst[c] = from_f32<T>(v);
            else dst[sp_k_index(off, c, Dp, k_tiled)] = from_f32<T>(v);
        };
        if (i < rh) {
            const float a = load(i), b = load(i + rh);
            store(i, a * cs[i] - b * sn[i]);
            store(i + rh, b * cs[i] + a * sn[i]);
        } else {
            const int c = rot + (i - rh);
            store(c, load(c));
        }
    }
    for (int it = tid; it < (qk_hi > h_lo ? qk_hi - h_lo : 0) * (Dp - D); it += WIDE_NT) {
        const int hh = h_lo + it / (Dp - D), c = D + it % (Dp - D);
        if (hh < HQ) q_out[((size_t)t * HQ + hh) * Dp + c] = from_f32<T>(0.f);
        else k_pages[(page * GK + (hh - HQ)) * (size_t)ps * Dp + sp_k_index(off, c, Dp, k_tiled)] = from_f32<T>(0.f);
    }
    if (slot < 0) return;
    const int vitems = Vd - vh;
    const int vbase = v_from_k ? Nq : Nq + Nk;           // the values are the keys as the row holds them (before their norm)
    for (int it = tid; it < (v_hi > v_lo ? v_hi - v_lo : 0) * vitems; it += WIDE_NT) {
        const int g = v_lo + it / vitems, i = it % vitems;
        T* slab = v_pages + (page * GV + g) * (size_t)Vd * ps;
        auto load = [&](int c) { return to_f32<T>(row[vbase + g * Vd + c]) + (bias ? bias[vbase + g * Vd + c] : 0.f); };
        if (i < vh) {
            const float a = load(i), b = load(i + vh);
            slab[sp_v_index(i, off, Vd, ps, v_tiled)] = from_f32<T>(a * csv[i] - b * snv[i]);
            slab[sp_v_index(i + vh, off, Vd, ps, v_tiled)] = from_f32<T>(b * csv[i] + a * snv[i]);
        } else {
            const int c = 2 * vh + (i - vh);
            slab[sp_v_index(c, off, Vd, ps, v_tiled)] = from_f32<T>(load(c));
        }
    }
}

// The same for bfloat16 rows whose sizes let a thread move four elements at a time (D, Dp, the row stride
// and the distance between a pair's elements multiples of four): 8-byte loads and stores for queries and
// keys (four elements in a row stay in a row in operand order too), the values one by one as above.  Every
// value is computed by the same operations as in the kernel above.
__global__ __launch_bounds__(WIDE_NT)
void qkv_prepare_vec_kernel(const bf16* __restrict__ qkv, int ld, const float* __restrict__ bias,
                            const float* __restrict__ wq, const float* __restrict__ wk, float eps,
                            bf16* __restrict__ q_out, bf16* __restrict__ k_pages, bf16* __restrict__ v_pages,
                            const int* __restrict__ positions, const int* __restrict__ slot_map,
                            const float* __restrict__ inv_freq, int rot, float rot_mag, const float* __restrict__ inv_freq_v,
                            int HQ, int GK, int GV, int D, int Vd, int ps, int k_tiled, int v_tiled, int Dp, int hpb,
                            int head_norm, float qt_coef, int qt_every, int v_from_k) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    __shared__ float red[WIDE_NT / 64];
    const int rh = rot >> 1, vh = inv_freq_v ? (Vd >> 1) : 0;
    float* cs = sm;
    float* sn = cs + rh;
    float* csv = sn + rh;
    float* snv = csv + vh;
    const int t = blockIdx.x, tid = threadIdx.x;
    const float pos = (float)positions[t];
    const bf16* row = qkv + (size_t)t * ld;
    const int Nq = HQ * D, Nk = GK * D;
    for (int i = tid; i < rh; i += WIDE_NT) { float sv, cv; sincosf(pos * inv_freq[i], &sv, &cv); sn[i] = sv * rot_mag; cs[i] = cv * rot_mag; }
    for (int i = tid; i < vh; i += WIDE_NT) sincosf(pos * inv_freq_v[i], &snv[i], &csv[i]);
    const int slot = slot_map ? slot_map[t] : -1;
    const int h_lo = blockIdx.y * hpb, h_end = h_lo + hpb;
    const int qk_end = HQ + (slot >= 0 ? GK : 0);
    const int qk_hi = h_end < qk_end ? h_end : qk_end;
    const int v_lo = (h_lo > HQ + GK ? h_lo : HQ + GK) - (HQ + GK);
    const int v_hi = (h_end < HQ + GK + GV ? h_end : HQ + GK + GV) - (HQ + GK);
    auto row4 = [&](int c) {                               // four elements of the row from c on, with their bias
        const bf16x4 r = *(const bf16x4*)(row + c);
        f32x4 x = {(float)r[0], (float)r[1], (float)r[2], (float)r[3]};
        if (bias) x += *(const f32x4*)(bias + c);
        return x;
    };
    auto sumsq = [&](int from, int n) {
        float s = 0.f;
        for (int c = tid * 4; c < n; c += WIDE_NT * 4) { const f32x4 x = row4(from + c); s += x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3]; }
        return block_sum<WIDE_NT>(s, red);
    };
    float scale_q = 1.f, scale_k = 1.f;
    __shared__ float head_sc[QKV_MAX_HPB];
    if (head_norm) {
        for (int hh = h_lo + (tid >> 6); hh < qk_hi; hh += WIDE_NT / 64) {
            float s = 0.f;
            for (int c = (tid & 63) * 4; c < D; c += 256) { const f32x4 x = row4(hh * D + c); s += x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3]; }
            s = wave_sum(s);
            if ((tid & 63) == 0) head_sc[hh - h_lo] = 1.0f / sqrtf(s / (float)D + eps);
        }
    }
    const float q_temp = qt_every > 0 ? 1.0f + qt_coef * logf((float)((positions[t] + 1) / qt_every) + 1.0f) : 1.0f;
    if (!head_norm && wq && h_lo < HQ) scale_q = 1.0f / sqrtf(sumsq(0, Nq) / (float)Nq + eps);
    if (!head_norm && wk && h_lo < qk_end && h_end > HQ) scale_k = 1.0f / sqrtf(sumsq(Nq, Nk) / (float)Nk + eps);
    __syncthreads();
    const size_t page = slot >= 0 ? (size_t)(slot / ps) : 0;
    const int off = slot >= 0 ? slot % ps : 0;
    // a head in groups of four: pairs that turn, elements that pass through, zeros behind D
    const int pq = rh >> 2, sq = (D - rot) >> 2, zq = (Dp - D) >> 2, QI = pq + sq + zq;
    const int n_qk = (qk_hi > h_lo ? qk_hi - h_lo : 0) * QI;
    for (int it = tid; it < n_qk; it += WIDE_NT) {
        const int hh = h_lo + it / QI, j = it % QI;
        const bool is_q = hh < HQ;
        const int base = hh * D;
        const float* wn = is_q ? wq : wk;
        const float sc = head_norm ? head_sc[hh - h_lo] : (is_q ? scale_q : scale_k);
        const int wbase = head_norm ? 0 : (is_q ? base : base - Nq);
        const float qt = is_q ? q_temp : 1.0f;
        auto load = [&](int c) {
            f32x4 x = row4(base + c);
            if (wn) { const f32x4 ww = *(const f32x4*)(wn + wbase + c); x = x * sc * ww; }
            return x * qt;
        };
        bf16* dst = is_q ? q_out + ((size_t)t * HQ + hh) * Dp : k_pages + (page * GK + (hh - HQ)) * (size_t)ps * Dp;
        auto store = [&](int c, const f32x4& v) {
            const bf16x4 o = {(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
            *(bf16x4*)(dst + (is_q ? (size_t)c : sp_k_index(off, c, Dp, k_tiled))) = o;
        };
        if (j < pq) {
            const int i = j * 4;
            const f32x4 a = load(i), b = load(i + rh);
            const f32x4 c4 = *(const f32x4*)(cs + i), s4 = *(const f32x4*)(sn + i);
            store(i, a * c4 - b * s4);
            store(i + rh, b * c4 + a * s4);
        } else if (j < pq + sq) {
            const int c = rot + (j - pq) * 4;
            store(c, load(c));
        } else {
            store(D + (j - pq - sq) * 4, f32x4{0.f, 0.f, 0.f, 0.f});
        }
    }
    if (slot < 0) return;
    const int vitems = Vd - vh;
    const int vbase = v_from_k ? Nq : Nq + Nk;
    for (int it = tid; it < (v_hi > v_lo ? v_hi - v_lo : 0) * vitems; it += WIDE_NT) {
        const int g = v_lo + it / vitems, i = it % vitems;
        bf16* slab = v_pages + (page * GV + g) * (size_t)Vd * ps;
        auto load = [&](int c) { return (float)row[vbase + g * Vd + c] + (bias ? bias[vbase + g * Vd + c] : 0.f); };
        if (i < vh) {
            const float a = load(i), b = load(i + vh);
            slab[sp_v_index(i, off, Vd, ps, v_tiled)] = (bf16)(a * csv[i] - b * snv[i]);
            slab[sp_v_index(i + vh, off, Vd, ps, v_tiled)] = (bf16)(b * csv[i] + a * snv[i]);
        } else {
            const int c = 2 * vh + (i - vh);
            slab[sp_v_index(c, off, Vd, ps, v_tiled)] = (bf16)load(c);
        }
    }
}

extern "C" int spite_qkv_prepare(const void* qkv, int ld, int dtype, const float* bias, const float* wq, const float* wk,
                                 float eps, void* q_out, void* k_pages, void* v_pages, const int* positions,
                                 const int* slot_map, const float* inv_freq, int rot, float rot_mag, const float* inv_freq_v,
                                 int T, int HQ, int GK, int GV, int D, int Vd, int page_size, int k_tiled, int v_tiled,
                                 int Dp, int head_norm, float qt_coef, int qt_every, int v_from_k, hipStream_t st) {
    if (Dp <= 0) Dp = D;
    SP_REQUIRE(Dp >= D, "qkv_prepare: heads of %d stored with %d elements", D, Dp);
    SP_REQUIRE(T >= 0 && HQ > 0 && GK > 0 && GV > 0 && D > 0 && Vd > 0 && page_size > 0, "qkv_prepare: bad sizes");
    SP_REQUIRE(ld >= (HQ + GK) * D + (v_from_k ? 0 : GV * Vd), "qkv_prepare: rows of %d elements for %d", ld, (HQ + GK) * D + (v_from_k ? 0 : GV * Vd));
    SP_REQUIRE(!v_from_k || (GV == GK && Vd == D && !inv_freq_v), "qkv_prepare: values taken from the keys have the keys' heads and width");
    SP_REQUIRE(!head_norm || (wq && wk), "qkv_prepare: a head norm needs its two weight vectors");
    SP_REQUIRE(qt_every >= 0, "qkv_prepare: query temperature every %d positions", qt_every);
    SP_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D, "qkv_prepare: %d turning elements of a head of %d", rot, D);
    SP_REQUIRE(rot == 0 || inv_freq, "qkv_prepare: rotation needs a frequency table");
    SP_REQUIRE(!inv_freq_v || Vd % 2 == 0, "qkv_prepare: values of %d elements cannot turn in pairs", Vd);
    SP_REQUIRE(!slot_map || (k_pages && v_pages), "qkv_prepare: writing the cache needs its pages");
    SP_REQUIRE(!k_tiled || (dtype == SP_BF16 && Dp % 32 == 0 && page_size % 32 == 0), "qkv_prepare: keys of %d in operand order", Dp);
    SP_REQUIRE(!v_tiled || (dtype == SP_BF16 && Vd % 32 == 0 && page_size % 32 == 0), "qkv_prepare: values of %d in operand order", Vd);
    SP_REQUIRE(eps > 0.f || (!wq && !wk), "qkv_prepare: the norm needs an eps");
    if (T == 0) return 0;
    const size_t sh = (size_t)(rot + (inv_freq_v ? Vd : 0)) * sizeof(float);
    SP_REQUIRE(sh <= 48 * 1024, "qkv_prepare: heads too wide");
    // heads a workgroup: all of a token's for many tokens; for few, so many that about two workgroups a compute unit run
    const int heads = HQ + GK + GV;
    long hpb = ((long)heads * T + 2 * sp_cu_count() - 1) / (2 * sp_cu_count());
    if (hpb < 1) hpb = 1;
    if (hpb > QKV_MAX_HPB) hpb = QKV_MAX_HPB;                          // (more waves in flight hide the rows' 2-byte loads and stores)
    if (hpb > heads) hpb = heads;
    const dim3 grid(T, (unsigned)((heads + hpb - 1) / hpb));
    auto al = [](const void* p, int a) { return ((uintptr_t)p & (a - 1)) == 0; };
    if (dtype == SP_BF16 && D % 4 == 0 && Dp % 4 == 0 && rot % 8 == 0 && ld % 4 == 0 && al(qkv, 8) && al(q_out, 8) && al(k_pages, 8)
        && al(bias, 16) && al(wq, 16) && al(wk, 16)) {
        // (the sine and cosine tables are read four at a time: the second starts rot/2 floats behind the first)
        qkv_prepare_vec_kernel<<<grid, WIDE_NT, sh, st>>>((const bf16*)qkv, ld, bias, wq, wk, eps, (bf16*)q_out, (bf16*)k_pages,
            (bf16*)v_pages, positions, slot_map, inv_freq, rot, rot_mag, inv_freq_v, HQ, GK, GV, D, Vd, page_size, k_tiled, v_tiled, Dp, (int)hpb, head_norm, qt_coef, qt_every, v_from_k);
        SP_LAUNCH_CHECK("qkv_prepare");
        return 0;
    }
    if (dtype == SP_F32)
        qkv_prepare_kernel<float><<<grid, WIDE_NT, sh, st>>>((const float*)qkv, ld, bias, wq, wk, eps, (float*)q_out, (float*)k_pages,
            (float*)v_pages, positions, slot_map, inv_freq, rot, rot_mag, inv_freq_v, HQ, GK, GV, D, Vd, page_size, k_tiled, v_tiled, Dp, (int)hpb, head_norm, qt_coef, qt_every, v_from_k);
    else if (dtype == SP_BF16)
        qkv_prepare_kernel<bf16><<<grid, WIDE_NT, sh, st>>>((const bf16*)qkv, ld, bias, wq, wk, eps, (bf16*)q_out, (bf16*)k_pages,
            (bf16*)v_pages, positions, slot_map, inv_freq, rot, rot_mag, inv_freq_v, HQ, GK, GV, D, Vd, page_size, k_tiled, v_tiled, Dp, (int)hpb, head_norm, qt_coef, qt_every, v_from_k);
    else return sp_fail("qkv_prepare: unknown dtype %d", dtype);
    SP_LAUNCH_CHECK("qkv_prepare");
    return 0;
}

// ------------------------------------------------------------------ the plain attention kernel
// One wave per (token, query head).  Keys are walked in tiles of 64 that start at the first
// visible key, so the order of every sum depends on the query's position alone: a token gives
// the same bits whether it comes in a whole prompt, a portion or alone.  With `sinks` (fp32 [HQ])
// every head's softmax has one more term in its denominator, exp(sinks[h]): a score that is not
// scaled, belongs to no key and brings no value.
#define WIDE_MAX_V 8   // value widths up to 512

template <typename T, typename TO>
__global__ __launch_bounds__(64)
void attn_wide_kernel(const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                      TO* __restrict__ out, const int* __restrict__ positions,
                      const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
                      int max_blocks, int HQ, int GK, int GV, int D, int Vd, int ps, int vis, int span, float scale,
                      int k_tiled, int v_tiled, const float* __restrict__ sinks, const float* __restrict__ slopes) {
    extern __shared__ float smem[];
    float* q_sh = smem;                 // [D]
    float* p_sh = smem + D;             // [64]
    int* page_sh = (int*)(p_sh + 64);   // [64] page of each key of the tile, -1 = none
    int* off_sh = page_sh + 64;         // [64] the key's offset in its page
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int g = h / (HQ / GK), gv = g % GV;
    const int p = positions[t];
    const int* bt = block_table + (size_t)seq_of_token[t] * max_blocks;
    const int lo = sp_first_visible(p, vis, span);
    const T* qr = q + ((size_t)t * HQ + h) * D;
    for (int c = lane; c < D; c += 64) q_sh[c] = to_f32<T>(qr[c]);
    __syncthreads();

    // the sink is the softmax's first term: it sets the running maximum and counts once
    float m = sinks ? sinks[h] : -INFINITY, l = sinks ? 1.f : 0.f;
    float o[WIDE_MAX_V];
#pragma unroll
    for (int u = 0; u < WIDE_MAX_V; ++u) o[u] = 0.f;

    for (int j0 = lo; j0 <= p; j0 += 64) {
        const int j = j0 + lane;
        float s = -INFINITY;
        int page = -1;
        if (j <= p) {
            page = bt[j / ps];
            if (page < 0) {
                s = NAN;   // a page that was given back is asked for: poison the result
            } else {
                const T* kr = k_pages + ((size_t)page * GK + g) * (size_t)ps * D;
                float acc = 0.f;
                for (int c = 0; c < D; ++c) acc = fmaf(q_sh[c], to_f32<T>(kr[sp_k_index(j % ps, c, D, k_tiled)]), acc);
                s = acc * scale;
                if (slopes) s += slopes[h] * (float)(j - p);       // a bias that grows with the distance
            }
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float alpha = expf(m - m_new);
        const float pj = (j <= p) ? expf(s - m_new) : 0.f;
        l = l * alpha + wave_sum(pj);
        m = m_new;
        __syncthreads();
        p_sh[lane] = pj;
        page_sh[lane] = page;
        off_sh[lane] = j % ps;
        __syncthreads();
        const int n_valid = (p - j0 + 1) < 64 ? (p - j0 + 1) : 64;
#pragma unroll
        for (int u = 0; u < WIDE_MAX_V; ++u) {
            const int c = lane + u * 64;
            if (c < Vd) {
                float acc = o[u] * alpha;
                for (int jj = 0; jj < n_valid; ++jj) {
                    const int pg = page_sh[jj];
                    const float vv = pg >= 0 ? to_f32<T>(v_pages[((size_t)pg * GV + gv) * (size_t)Vd * ps + sp_v_index(c, off_sh[jj], Vd, ps, v_tiled)]) : 0.f;
                    acc = fmaf(p_sh[jj], vv, acc);
                }
                o[u] = acc;
            }
        }
    }
    const float inv = 1.0f / fmaxf(l, 1e-30f);
    TO* orow = out + ((size_t)t * HQ + h) * Vd;
#pragma unroll
    for (int u = 0; u < WIDE_MAX_V; ++u) {
        const int c = lane + u * 64;
        if (c < Vd) orow[c] = from_f32<TO>(o[u] * inv);
    }
}

extern "C" int spite_attn_wide(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype, int out_dtype,
                               const int* positions, const int* seq_of_token, const int* block_table,
                               int max_blocks, int T, int HQ, int GK, int GV, int D, int Vd, int page_size, int vis, int span,
                               float scale, int k_tiled, int v_tiled, const float* sinks, const float* slopes, hipStream_t st) {
    SP_REQUIRE(T >= 0 && HQ > 0 && GK > 0 && GV > 0 && HQ % GK == 0 && GK % GV == 0,
               "attention: %d query heads over %d key heads over %d value heads", HQ, GK, GV);
    SP_REQUIRE(D > 0 && D <= 4096 && Vd > 0 && Vd <= 64 * WIDE_MAX_V, "attention: keys of %d, values of %d (at most %d)", D, Vd, 64 * WIDE_MAX_V);
    SP_REQUIRE(page_size > 0 && max_blocks > 0, "attention: bad page size %d or table width %d", page_size, max_blocks);
    SP_REQUIRE(vis >= 0 && vis < SP_VIS_COUNT && (!sp_vis_has_span(vis) || span > 0), "attention: chunk or window of %d", span);
    SP_REQUIRE(HQ <= 65535, "attention: too many heads");
    SP_REQUIRE(!k_tiled || (dtype == SP_BF16 && D % 32 == 0 && page_size % 32 == 0), "attention: keys of %d in operand order", D);
    SP_REQUIRE(!v_tiled || (dtype == SP_BF16 && Vd % 32 == 0 && page_size % 32 == 0), "attention: values of %d in operand order", Vd);
    if (T == 0) return 0;
    dim3 grid(T, HQ);
    const size_t sh = (size_t)(D + 64) * sizeof(float) + 128 * sizeof(int);
#define SP_AW(TI, TO) attn_wide_kernel<TI, TO><<<grid, 64, sh, st>>>((const TI*)q, (const TI*)k_pages, (const TI*)v_pages, (TO*)out, \
        positions, seq_of_token, block_table, max_blocks, HQ, GK, GV, D, Vd, page_size, vis, span, scale, k_tiled, v_tiled, sinks, slopes)
    if (dtype == SP_F32 && out_dtype == SP_F32) SP_AW(float, float);
    else if (dtype == SP_BF16 && out_dtype == SP_BF16) SP_AW(bf16, bf16);
    else if (dtype == SP_BF16 && out_dtype == SP_F32) SP_AW(bf16, float);
    else return sp_fail("attention: dtypes %d -> %d", dtype, out_dtype);
#undef SP_AW
    SP_LAUNCH_CHECK("attn_wide");
    return 0;
}

// ------------------------------------------------------------------ attention result -> output projection's operand
// One wave per (token, head).  in [T, maps*H, Vd] (map by map), out [T, H*Vd].
//   maps == 2:      o = a1 - lambda * a2, then o / sqrt(mean(o^2) + eps) * post   (over the head's Vd values)
//   inv_freq_v:     pairs (m, m + Vd/2) of o turn by -pos * inv_freq_v[m]
//   gate:           o *= sigmoid(gate[t*ldg + h])
template <typename TI, typename TG, typename TO>
__global__ __launch_bounds__(64)
void attn_finish_kernel(const TI* __restrict__ in, TO* __restrict__ out, const int* __restrict__ positions,
                        const float* __restrict__ inv_freq_v, const TG* __restrict__ gate, int ldg,
                        int H, int Vd, int maps, float lambda, float eps, float post) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const TI* a1 = in + ((size_t)t * maps * H + h) * Vd;
    TO* orow = out + ((size_t)t * H + h) * Vd;
    float g = 1.f;
    if (gate) g = 1.0f / (1.0f + expf(-to_f32<TG>(gate[(size_t)t * ldg + h])));
    if (maps == 2) {
        const TI* a2 = a1 + (size_t)H * Vd;
        float ss = 0.f;
        for (int c = lane; c < Vd; c += 64) { const float o = to_f32<TI>(a1[c]) - lambda * to_f32<TI>(a2[c]); ss += o * o; }
        const float sc = post / sqrtf(wave_sum(ss) / (float)Vd + eps) * g;
        for (int c = lane; c < Vd; c += 64) orow[c] = from_f32<TO>((to_f32<TI>(a1[c]) - lambda * to_f32<TI>(a2[c])) * sc);
        return;
    }
    if (inv_freq_v) {
        const int vh = Vd >> 1;
        const float pos = (float)positions[t];
        for (int i = lane; i < vh; i += 64) {
            float s, c;
            sincosf(pos * inv_freq_v[i], &s, &c);
            const float a = to_f32<TI>(a1[i]), b = to_f32<TI>(a1[i + vh]);
            orow[i] = from_f32<TO>((a * c + b * s) * g);          // the turn by -angle
            orow[i + vh] = from_f32<TO>((b * c - a * s) * g);
        }
        return;
    }
    for (int c = lane; c < Vd; c += 64) orow[c] = from_f32<TO>(to_f32<TI>(a1[c]) * g);
}

extern "C" int spite_attn_finish(const void* in, int in_dtype, void* out, int out_dtype, const int* positions,
                                 const float* inv_freq_v, const void* gate, int ldg, int T, int H, int Vd, int maps,
                                 float lambda, float eps, float post, hipStream_t st) {
    SP_REQUIRE(T >= 0 && H > 0 && H <= 65535 && Vd > 0, "attn_finish: bad sizes");
    SP_REQUIRE(maps == 1 || maps == 2, "attn_finish: %d score maps a head", maps);
    SP_REQUIRE(maps == 1 || (eps > 0.f && !inv_freq_v), "attn_finish: two maps are normed (eps) and not turned");
    SP_REQUIRE(!inv_freq_v || (Vd % 2 == 0 && positions), "attn_finish: values of %d cannot turn in pairs", Vd);
    SP_REQUIRE(!gate || ldg >= H, "attn_finish: gate rows of %d for %d heads", ldg, H);
    if (T == 0) return 0;
    dim3 grid(T, H);
    // the gate comes from the run's projection, so it has the output's type
#define SP_AF(TI, TO) attn_finish_kernel<TI, TO, TO><<<grid, 64, 0, st>>>((const TI*)in, (TO*)out, positions, inv_freq_v, \
        (const TO*)gate, ldg, H, Vd, maps, lambda, eps, post)
    if (in_dtype == SP_F32 && out_dtype == SP_F32) SP_AF(float, float);
    else if (in_dtype == SP_F32 && out_dtype == SP_BF16) SP_AF(float, bf16);
    else if (in_dtype == SP_BF16 && out_dtype == SP_BF16) SP_AF(bf16, bf16);
    else return sp_fail("attn_finish: dtypes %d -> %d", in_dtype, out_dtype);
#undef SP_AF
    SP_LAUNCH_CHECK("attn_finish");
    return 0;
}
