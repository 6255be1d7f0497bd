// The one-token attention of the decode step as a device function: shared by the stand-alone decode
// kernels and by the kernels that run the attention next to the projections around it.
#pragma once
#include <cfloat>
#include <cmath>

#include "common.hpp"

#define AD_THREADS 512
#define AD_WAVES 8
#define AD_MAX_SPLITS 256
#define AD_LS 512 // positions per span (longest)

struct AdArgs {
    const half_t *q;   // plain: rotated queries [Hq*hd]; fused: the raw qkv row [(Hq+2Hkv)*hd]
    half_t *kc, *vc;   // caches of this layer
    half_t *out;       // [Hq*hd]
    const float *table; // fused: (cos, sin) table [max_pos][hd/2][2]
    int pos_host;
    const int32_t *pos_dev; // position of the new token = pos_host + *pos_dev; ctx = position + 1
    int n_kv_heads, max_pos, splits;
    int span_target;   // long form: spans per kv head that give every CU one (CUs / kv heads, 1..64)
    float *ws_acc, *ws_ml;
    int *counters;
};

// Long form: positions per span and number of spans of a context of ctx positions.  256 positions per span (eight
// wavefronts of 32) once that makes at least `target` spans per kv head (target = CUs per kv head: every CU has a
// span workgroup); shorter contexts are cut into spans of 128 or 64 positions, whose workgroups leave wavefronts
// idle but spread the cache rows over more CUs.  Two span workgroups fit a CU, so up to 2 * CUs of them run side
// by side.  (Measured against spans cut for exactly one workgroup per CU, sixteen wavefronts each: those were
// 0.4 to 1.6 us slower per launch at 2K to 16K positions.)
__host__ __device__ inline int ad_long_span(int ctx, int target) {
    int s = 256;
    while (s > 64 && (ctx + s - 1) / s < target) s >>= 1;
    return s;
}
__host__ __device__ inline int ad_long_spans(int ctx, int target) {
    const int s = ad_long_span(ctx, target);
    return (ctx + s - 1) / s;
}
// spans of any context up to max_pos: ceil(max_pos / 256) with the longest spans, fewer than 2 * target with shorter ones
__host__ __device__ inline int ad_long_max_spans(int max_pos, int target) {
    int n = (max_pos + 255) / 256;
    if (2 * target - 2 > n) n = 2 * target - 2;
    const int cap = (max_pos + 63) / 64;
    if (n > cap) n = cap;
    return n < 1 ? 1 : n;
}

// Every K and V load of the span is issued before anything else (a span is at
// most 512 positions: 16 + 2..16 loads of 16 bytes per thread at hd 128), so the
// whole span costs one trip to HBM instead of one per loop iteration.  In the
// fused form the new token's own K and V come from the projection row through
// LDS (and are written to the cache for later steps), so nothing waits on
// that write.
//
// NDIM is the number of head dims this workgroup produces, LS the span length.

// LDS of the attention.  The K staging buffer depends on the head size only: a kernel that instantiates the body
// twice (for a quarter of the dims and for all of them) holds it once.
template <int HD> __device__ __forceinline__ half_t *ad_lds_kst() {
    __shared__ __attribute__((aligned(16))) half_t buf[AD_WAVES * 32 * (HD + 8)];
    return buf;
}
template <int NDIM, int G> __device__ __forceinline__ float *ad_lds_ow() {
    __shared__ __attribute__((aligned(16))) float buf[AD_WAVES * G * NDIM];
    return buf;
}
template <int G> __device__ __forceinline__ float *ad_lds_ml() {
    __shared__ float buf[AD_WAVES * G * 2];
    return buf;
}

// One span of at most NB * 256 positions.  Wavefront w owns the 32-position blocks [256 c + 32 w, + 32), c < NB,
// and runs the whole attention on them by itself, on the matrix pipe:
//   scores   S[pos][head] = K_block . q^T    (v_mfma_f32_16x16x32_f16, K rows as the row operand, the group's
//            queries as columns 0..G-1), with the K rows of the two 16-row halves interleaved so that a lane
//            ends up with eight consecutive positions of one head: the layout of the next product's operand;
//   softmax  relative to the wavefront's own maximum, in registers (reductions over four lanes);
//   P.V      O[dim][head] += V_block^T . P   (the V cache is dim-major: a lane's operand is one 16-byte load).
// What the wavefronts leave (maximum, sum, unnormalised O) is combined once through LDS.  Two workgroup barriers
// in all, both on LDS contents only, so the cache-row loads stay in flight across the first.
// Every cache-row load is issued unconditionally (positions beyond the span re-read its last row and are masked
// afterwards): with a fixed number of loads in flight the waits can name the loads they need, and the rotation
// of the new token, whose inputs are requested first, runs while the cache rows are still on their way.
template <int HD, int G, bool FUSED, int NDIM, int LS, bool AGENT_OUT, int NB>
__device__ __forceinline__ void attn_decode_span(const AdArgs &a, half_t *qs, half_t *knew, half_t *vnew,
                                                 half_t *kst_all, float *ow_all, float *ml_all, const int pos,
                                                 const int n_active, const int split, const int d_begin,
                                                 const bool appender, const int kvh) {
    constexpr int LPP = HD / 8;   // lanes per K row
    constexpr int PPW = 64 / LPP; // K rows per load instruction of a wavefront
    constexpr int NPB = 32 / PPW; // load instructions per block
    constexpr int KS = HD / 32;   // k-steps of the score product
    constexpr int NT = NDIM / 16; // 16-dim tiles of the output
    constexpr int KLD = HD + 8;   // row stride of the staging slice (halves): fragment reads without bank conflicts
    constexpr int HALF = HD / 2;
    static_assert(HD % 32 == 0 && NDIM % 16 == 0 && G <= 16 && NB * 256 <= LS, "attention tiling");
    static_assert(G * HD <= AD_THREADS * 8 && G * NDIM / 4 <= AD_THREADS, "one staging / result item per thread");

    const int splits = a.splits;
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int max_pos = a.max_pos;
    const int ctx = pos + 1;
    const int s0 = split * LS;
    const int len = ctx - s0 < LS ? ctx - s0 : LS;
    half_t *kbase = a.kc + (size_t)kvh * max_pos * HD;
    half_t *vrow0 = a.vc + (size_t)kvh * HD * max_pos;
    const int lpos = pos - s0; // the new token inside this span (last span only)
    const int mg = lane / 16, mn = lane % 16;
    const int sub = lane % LPP, prow = lane / LPP;
    const int blk0 = 32 * wave; // first position of this wavefront's block c is 256 c + blk0

    // ---- 0. the new token's inputs, requested before the cache rows -----------------------
    constexpr int NRI = ((G + 1) * HALF + AD_THREADS - 1) / AD_THREADS; // rotation pairs per thread
    constexpr int NVI = (HD + AD_THREADS - 1) / AD_THREADS;             // new-v elements per thread
    uint32_t pair_r[NRI];
    float2_t cs_r[NRI];
    half_t vnew_r[NVI];
    half8_t q_r = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    if (FUSED) {
        const int Hq = a.n_kv_heads * G;
        const float *cs = a.table + (size_t)pos * HALF * 2;
#pragma unroll
        for (int r = 0; r < NRI; ++r) {
            const int p = tid + r * AD_THREADS;
            if (p < (G + 1) * HALF) {
                const int h = p / HALF, i = p % HALF; // h == G: the new key
                const half_t *src = h < G ? a.q + (size_t)(kvh * G + h) * HD + 2 * i
                                          : a.q + (size_t)Hq * HD + (size_t)kvh * HD + 2 * i;
                pair_r[r] = *reinterpret_cast<const uint32_t *>(src);
                cs_r[r] = *reinterpret_cast<const float2_t *>(cs + 2 * i);
            }
        }
#pragma unroll
        for (int r = 0; r < NVI; ++r) {
            const int d = tid + r * AD_THREADS;
            if (d < HD) vnew_r[r] = a.q[(size_t)(Hq + a.n_kv_heads) * HD + (size_t)kvh * HD + d];
        }
    }
    if (!FUSED && tid * 8 < G * HD) q_r = load8(a.q + (size_t)kvh * G * HD + tid * 8);

    // ---- 1. every K and V load of the wavefront's blocks -----------------------------------
    half8_t kreg[NB][NPB];
#pragma unroll
    for (int c = 0; c < NB; ++c) {
#pragma unroll
        for (int q = 0; q < NPB; ++q) {
            const int j = 256 * c + blk0 + q * PPW + prow;
            const int jc = j < len ? j : len - 1;
            kreg[c][q] = load8(kbase + (size_t)(s0 + jc) * HD + sub * 8);
        }
    }
    half8_t vreg[NB][NT]; // lane (mg, mn): dim 16 t + mn, positions 8 mg .. + 7 of the block
#pragma unroll
    for (int c = 0; c < NB; ++c) {
        const int j = 256 * c + blk0 + 8 * mg;
        const int jc = j < len ? j : ((len - 1) & ~7);
#pragma unroll
        for (int t = 0; t < NT; ++t)
            vreg[c][t] = load8(vrow0 + (size_t)(d_begin + 16 * t + mn) * max_pos + s0 + jc);
    }

    // ---- 2. queries into LDS; fused: rotate them and the new K, append K/V ---------
    if (FUSED) {
#pragma unroll
        for (int r = 0; r < NRI; ++r) {
            const int p = tid + r * AD_THREADS;
            if (p < (G + 1) * HALF) {
                const int h = p / HALF, i = p % HALF; // h == G: the new key
                const half2_t pr = __builtin_bit_cast(half2_t, pair_r[r]);
                const float c = cs_r[r][0], sn = cs_r[r][1], e = (float)pr[0], o = (float)pr[1];
                const float ce = c * e, so = sn * o, se = sn * e, co = c * o;
                const half_t re = (half_t)(ce - so), ro = (half_t)(se + co);
                if (h < G) {
                    qs[h * HD + 2 * i] = re;
                    qs[h * HD + 2 * i + 1] = ro;
                } else {
                    knew[2 * i] = re;
                    knew[2 * i + 1] = ro;
                    if (appender) {
                        kbase[(size_t)pos * HD + 2 * i] = re;
                        kbase[(size_t)pos * HD + 2 * i + 1] = ro;
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < NVI; ++r) {
            const int d = tid + r * AD_THREADS;
            if (d < HD) {
                const half_t v = vnew_r[r];
                vnew[d] = v;
                if (appender) vrow0[(size_t)d * max_pos + pos] = v;
            }
        }
    } else {
        if (tid * 8 < G * HD) store8(qs + tid * 8, q_r);
    }
    // This barrier guards LDS contents only (queries, new key and value): it waits for the LDS writes and leaves
    // the cache-row loads in flight, which __syncthreads() would drain first.
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // ---- 3. scores of this wavefront's blocks -------------------------------------------
    // The K registers keep the row-contiguous load pattern (whole rows per position); the wavefront turns a block
    // into the MFMA's row operand through its own slice of LDS.  Row m of half u of the product is block row
    // 8 (m / 4) + 4 u + m % 4, so that lane (mg, mn) ends up with positions 8 mg .. + 7 of the block for head mn.
    half_t *kst = kst_all + wave * 32 * KLD;
    half8_t qreg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        qreg[ks] = mn < G ? load8(qs + mn * HD + 32 * ks + 8 * mg) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    const float scale = 1.0f / sqrtf((float)HD);
    float sv[NB][8];
#pragma unroll
    for (int c = 0; c < NB; ++c) {
#pragma unroll
        for (int q = 0; q < NPB; ++q) {
            const int r = q * PPW + prow;
            half8_t kv = kreg[c][q];
            if (FUSED && 256 * c + blk0 + r == lpos) kv = load8(knew + sub * 8);
            store8(kst + r * KLD + sub * 8, kv);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int row = 8 * (mn / 4) + 4 * u + mn % 4;
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(load8(kst + row * KLD + 32 * ks + 8 * mg), qreg[ks], acc, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = 256 * c + blk0 + 8 * mg + 4 * u + i;
                sv[c][4 * u + i] = j < len ? acc[i] * scale : -FLT_MAX;
            }
        }
    }

    // ---- 4. softmax relative to the wavefront's own maximum ------------------------------
    float m_w = -FLT_MAX;
#pragma unroll
    for (int c = 0; c < NB; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e) m_w = fmaxf(m_w, sv[c][e]);
    m_w = rows_max(m_w);
    float l_w = 0.f;
    half8_t pf[NB];
#pragma unroll
    for (int c = 0; c < NB; ++c) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int j = 256 * c + blk0 + 8 * mg + e;
            const float p = j < len ? __expf(sv[c][e] - m_w) : 0.f;
            l_w += p;
            pf[c][e] = (half_t)p;
        }
    }
    l_w = rows_sum(l_w);

    // ---- 5. unnormalised P.V of the blocks -------------------------------------------------
    float *ow = ow_all + wave * G * NDIM;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        float4_t o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NB; ++c) {
            const int j = 256 * c + blk0 + 8 * mg;
            half8_t vf = vreg[c][t];
            if (FUSED && lpos >= j && lpos < j + 8) { // the chunk that holds the new token
                const half_t vn = vnew[d_begin + 16 * t + mn];
#pragma unroll
                for (int e = 0; e < 8; ++e) vf[e] = (j + e == lpos) ? vn : vf[e];
            }
            if (j + 8 > len) { // beyond or across the end of the span
#pragma unroll
                for (int e = 0; e < 8; ++e) vf[e] = (j + e < len) ? vf[e] : (half_t)0.f;
            }
            o = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf[c], o, 0, 0, 0);
        }
        if (mn < G) *reinterpret_cast<float4_t *>(ow + mn * NDIM + 16 * t + 4 * mg) = o; // dims 16 t + 4 mg .. + 3
    }
    if (mn < G && mg == 0) {
        ml_all[(wave * G + mn) * 2] = m_w;
        ml_all[(wave * G + mn) * 2 + 1] = l_w;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // ---- 6. the wavefronts' parts into one: four dims of one head per thread ---------------------
    if (tid < G * NDIM / 4) {
        const int h = tid / (NDIM / 4), d4 = tid % (NDIM / 4);
        float mw[AD_WAVES];
        float M = -FLT_MAX;
#pragma unroll
        for (int w = 0; w < AD_WAVES; ++w) {
            mw[w] = ml_all[(w * G + h) * 2];
            M = fmaxf(M, mw[w]);
        }
        float L = 0.f;
        float4_t O = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < AD_WAVES; ++w) {
            const float f = __expf(mw[w] - M); // 0 for a wavefront without a position of the span
            L += f * ml_all[(w * G + h) * 2 + 1];
            const float4_t part = *reinterpret_cast<const float4_t *>(ow_all + (w * G + h) * NDIM + 4 * d4);
#pragma unroll
            for (int i = 0; i < 4; ++i) O[i] += f * part[i];
        }
        if (n_active == 1) {
            half_t *dst = a.out + (size_t)(kvh * G + h) * HD + d_begin + 4 * d4;
            if (AGENT_OUT) {
                // 8-byte device-scope stores (written through to the point where every XCD reads them): 2-byte
                // write-through stores cost a read-modify-write each
                unsigned long long v = 0ull;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    uint16_t bits = __builtin_bit_cast(uint16_t, (half_t)(O[i] / L));
                    if (bits == 0xFFFFu) bits = 0xFFFEu; // 0xFFFF marks "not written yet" for the reader
                    v |= (unsigned long long)bits << (16 * i);
                }
                __hip_atomic_store(reinterpret_cast<unsigned long long *>(dst), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) dst[i] = (half_t)(O[i] / L);
            }
        } else {
            float *dst = a.ws_acc + (((size_t)kvh * splits + split) * G + h) * HD + d_begin + 4 * d4;
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[i] = O[i];
            if (d4 == 0) {
                a.ws_ml[(((size_t)kvh * splits + split) * G + h) * 2 + 0] = M;
                a.ws_ml[(((size_t)kvh * splits + split) * G + h) * 2 + 1] = L;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
// Long contexts: one span of up to 256 positions per workgroup of eight wavefronts, every wavefront on its own
// (32 positions) until the final combine.
//
// The form above stages the rotated queries through LDS behind a workgroup barrier; with thousands of cached
// positions that barrier sits behind the issue of every cache-row load of the workgroup (the memory pipeline
// takes them in only as fast as data comes back), so nothing is computed before the last load has been handed
// over.  Here a wavefront asks for the raw queries of its kv group and their rotation entries first (spread over
// the lanes: lane (mg, mn) takes eight elements of head mn % G), then for its 32 key rows and its value rows,
// rotates the queries in registers while those are on their way, moves them across lanes into the score
// product's operand, and runs scores, softmax and P.V as the data lands; the first and only workgroup barrier
// stands in front of the combine of the wavefronts' (max, sum, P.V).  The arithmetic is that of
// attn_decode_span, step for step (same products, same order, same roundings).
// LAST: the span that ends with the new token (rotate its key, splice key and value into the registers of the
// wavefront that owns the position, append both to the caches); the other spans do not touch the new token.
// K and V rows are read once per step: non-temporal loads.
// LDS: one slice per wavefront (32 staged key rows, then reused for the wavefront's P.V; HD halves for the new
// value) + the (max, sum) pairs: 72 KB at head size 128 and at most 128 vector registers, so two workgroups share a CU.
#define AD_SPAN_WAVES 8
#define AD_SPAN_THREADS (64 * AD_SPAN_WAVES)
#define AD_SPAN 256 // positions per span of the long form, at most

template <int HD> __device__ __forceinline__ half_t *ad_lds_wave_slices() {
    __shared__ __attribute__((aligned(16))) half_t buf[AD_SPAN_WAVES * (32 * (HD + 8) + HD)];
    return buf;
}
template <int G> __device__ __forceinline__ float *ad_lds_span_ml() {
    __shared__ float buf[AD_SPAN_WAVES * G * 2];
    return buf;
}

template <int HD, int G, bool LAST>
__device__ __forceinline__ void attn_span_wave(const AdArgs &a, const int pos, const int split, const int kvh, const int span) {
    constexpr int LPP = HD / 8;   // lanes per K row
    constexpr int PPW = 64 / LPP; // K rows per load instruction of a wavefront
    constexpr int NPB = 32 / PPW; // load instructions per block
    constexpr int KS = HD / 32;   // k-steps of the score product
    constexpr int NT = HD / 16;   // 16-dim tiles of the output
    constexpr int KLD = HD + 8;   // row stride of the staging slice (halves)
    constexpr int HALF = HD / 2;
    constexpr int SLICE = 32 * KLD + HD;
    constexpr int QPP = 16 / G;                  // k-steps of the queries that the 16 lanes of a row cover in one pass
    constexpr int QPASS = (KS + QPP - 1) / QPP;
    static_assert(HD % 32 == 0 && 16 % G == 0 && G * HD * sizeof(float) <= 32 * KLD * sizeof(half_t), "attention tiling");
    static_assert(G * HD / 4 <= AD_SPAN_THREADS, "one result item per thread");

    const int splits = a.splits;
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int max_pos = a.max_pos;
    const int s0 = split * span; // span: 64, 128 or 256
    const int len = pos + 1 - s0 < span ? pos + 1 - s0 : span;
    half_t *kbase = a.kc + (size_t)kvh * max_pos * HD;
    half_t *vrow0 = a.vc + (size_t)kvh * HD * max_pos;
    const int mg = lane / 16, mn = lane % 16;
    const int sub = lane % LPP, prow = lane / LPP;
    const int blk0 = 32 * wave;
    const int lpos = pos - s0;                   // LAST: the new token inside this span
    const bool live = blk0 < len;                // wave-uniform: this wavefront has positions of the span
    const bool owner = LAST && lpos >= blk0 && lpos < blk0 + 32; // wave-uniform
    half_t *slice = ad_lds_wave_slices<HD>() + wave * SLICE;
    half_t *kst = slice, *vn_l = slice + 32 * KLD;
    float *ow = reinterpret_cast<float *>(slice); // the wavefront's P.V, once its key rows have been consumed
    float *ml_all = ad_lds_span_ml<G>();
    const int Hq = a.n_kv_heads * G;

    float m_w = -FLT_MAX, l_w = 0.f;
    if (live) {
        // ---- 0. raw queries of the group with their rotation entries, the new token's key and value ------
        const float *cs = a.table + (size_t)pos * HALF * 2;
        // pass p: lane (mg, mn) takes elements 32 ks + 8 mg .. + 7 of head mn % G, ks = p * QPP + mn / G
        half8_t q_raw[QPASS];
        float4_t q_cs[QPASS][2];
#pragma unroll
        for (int p = 0; p < QPASS; ++p) {
            const int ks = p * QPP + mn / G;
            q_raw[p] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
            q_cs[p][0] = q_cs[p][1] = float4_t{0, 0, 0, 0};
            if (ks < KS) {
                const int e0 = 32 * ks + 8 * mg;
                q_raw[p] = load8(a.q + (size_t)(kvh * G + mn % G) * HD + e0);
                q_cs[p][0] = *reinterpret_cast<const float4_t *>(cs + e0);
                q_cs[p][1] = *reinterpret_cast<const float4_t *>(cs + e0 + 4);
            }
        }
        half8_t k_raw = half8_t{0, 0, 0, 0, 0, 0, 0, 0}, v_raw = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        float4_t k_cs[2] = {float4_t{0, 0, 0, 0}, float4_t{0, 0, 0, 0}};
        if (LAST) {
            k_raw = load8(a.q + (size_t)Hq * HD + (size_t)kvh * HD + sub * 8);
            k_cs[0] = *reinterpret_cast<const float4_t *>(cs + sub * 8);
            k_cs[1] = *reinterpret_cast<const float4_t *>(cs + sub * 8 + 4);
            if (lane < HD / 8) v_raw = load8(a.q + (size_t)(Hq + a.n_kv_heads) * HD + (size_t)kvh * HD + lane * 8);
        }
        // ---- 1. the block's key rows (positions beyond the span re-read its last row and are masked later) ----
        half8_t kreg[NPB];
#pragma unroll
        for (int q = 0; q < NPB; ++q) {
            const int j = blk0 + q * PPW + prow;
            const int jc = j < len ? j : len - 1;
            kreg[q] = load8_nt(kbase + (size_t)(s0 + jc) * HD + sub * 8);
        }
        // ---- 2. the block's value rows: lane (mg, mn) holds dim 16 t + mn, positions 8 mg .. + 7 -------
        half8_t vreg[NT];
        {
            const int j = blk0 + 8 * mg;
            const int jc = j < len ? j : ((len - 1) & ~7);
#pragma unroll
            for (int t = 0; t < NT; ++t) vreg[t] = load8_nt(vrow0 + (size_t)(16 * t + mn) * max_pos + s0 + jc);
        }
        // ---- 3. queries rotated in registers, then across lanes into the B operand of the score product --
        // pair (x[2i], x[2i+1]) of a head by the angle of (pos, i): (c e - s o, s e + c o), rounded to fp16
        auto rotate8 = [](half8_t raw, float4_t c0, float4_t c1) {
            half8_t r;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const float c = p < 2 ? c0[2 * p] : c1[2 * p - 4], sn = p < 2 ? c0[2 * p + 1] : c1[2 * p - 3];
                const float e = (float)raw[2 * p], o = (float)raw[2 * p + 1];
                const float ce = c * e, so = sn * o, se = sn * e, co = c * o;
                r[2 * p] = (half_t)(ce - so);
                r[2 * p + 1] = (half_t)(se + co);
            }
            return r;
        };
        uint4_t q_rot[QPASS];
#pragma unroll
        for (int p = 0; p < QPASS; ++p) q_rot[p] = __builtin_bit_cast(uint4_t, rotate8(q_raw[p], q_cs[p][0], q_cs[p][1]));
        // lane (mg, mn < G) needs elements 32 ks + 8 mg .. + 7 of head mn for every ks: held by lane (mg, (ks % QPP) * G + mn)
        half8_t qreg[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int src = mn < G ? 16 * mg + (ks % QPP) * G + mn : lane;
            uint4_t v;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = (uint32_t)__builtin_amdgcn_ds_bpermute(4 * src, (int)q_rot[ks / QPP][i]);
            qreg[ks] = mn < G ? __builtin_bit_cast(half8_t, v) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }
        half8_t knew8 = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        if (LAST) {
            knew8 = rotate8(k_raw, k_cs[0], k_cs[1]);
            if (lane < HD / 8) store8(vn_l + lane * 8, v_raw);
        }
        // the new token's key row and value column into the caches, from the wavefront that owns the position
        if (owner) {
#pragma unroll
            for (int q = 0; q < NPB; ++q)
                if (blk0 + q * PPW + prow == lpos) store8(kbase + (size_t)pos * HD + sub * 8, knew8);
            if (lane < HD / 8) {
#pragma unroll
                for (int e = 0; e < 8; ++e) vrow0[(size_t)(lane * 8 + e) * max_pos + pos] = v_raw[e];
            }
        }
        // ---- 4. scores: K rows through the wavefront's own LDS slice into the MFMA's row operand --------
        const float scale = 1.0f / sqrtf((float)HD);
        float sv[8];
#pragma unroll
        for (int q = 0; q < NPB; ++q) {
            const int r = q * PPW + prow;
            half8_t kv = kreg[q];
            if (LAST && blk0 + r == lpos) kv = knew8;
            store8(kst + r * KLD + sub * 8, kv);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int row = 8 * (mn / 4) + 4 * u + mn % 4;
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(load8(kst + row * KLD + 32 * ks + 8 * mg), qreg[ks], acc, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = blk0 + 8 * mg + 4 * u + i;
                sv[4 * u + i] = j < len ? acc[i] * scale : -FLT_MAX;
            }
        }
        // ---- 5. softmax relative to the wavefront's own maximum ----------------------------------------
#pragma unroll
        for (int e = 0; e < 8; ++e) m_w = fmaxf(m_w, sv[e]);
        m_w = rows_max(m_w);
        half8_t pf;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int j = blk0 + 8 * mg + e;
            const float p = j < len ? __expf(sv[e] - m_w) : 0.f;
            l_w += p;
            pf[e] = (half_t)p;
        }
        l_w = rows_sum(l_w);
        // ---- 6. unnormalised P.V into the wavefront's slice (its key rows have been consumed) ----------
        float4_t o[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int j = blk0 + 8 * mg;
            half8_t vf = vreg[t];
            if (LAST && lpos >= j && lpos < j + 8) { // the chunk that holds the new token
                const half_t vn = vn_l[16 * t + mn];
#pragma unroll
                for (int e = 0; e < 8; ++e) vf[e] = (j + e == lpos) ? vn : vf[e];
            }
            if (j + 8 > len) { // beyond or across the end of the span
#pragma unroll
                for (int e = 0; e < 8; ++e) vf[e] = (j + e < len) ? vf[e] : (half_t)0.f;
            }
            o[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf, float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < NT; ++t)
            if (mn < G) *reinterpret_cast<float4_t *>(ow + mn * HD + 16 * t + 4 * mg) = o[t]; // dims 16 t + 4 mg .. + 3
    }
    if (mn < G && mg == 0) {
        ml_all[(wave * G + mn) * 2] = m_w;
        ml_all[(wave * G + mn) * 2 + 1] = l_w;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // ---- 7. the wavefronts' parts into one: four dims of one head per thread -----------------------------
    if (tid < G * HD / 4) {
        const int h = tid / (HD / 4), d4 = tid % (HD / 4);
        float mw[AD_SPAN_WAVES];
        float M = -FLT_MAX;
#pragma unroll
        for (int w = 0; w < AD_SPAN_WAVES; ++w) {
            mw[w] = ml_all[(w * G + h) * 2];
            M = fmaxf(M, mw[w]);
        }
        float L = 0.f;
        float4_t O = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < AD_SPAN_WAVES; ++w) {
            if (32 * w < len) { // wavefronts without a position of the span left nothing in their slice
                const float f = __expf(mw[w] - M);
                L += f * ml_all[(w * G + h) * 2 + 1];
                const float4_t part = *reinterpret_cast<const float4_t *>(
                    reinterpret_cast<const float *>(ad_lds_wave_slices<HD>() + w * SLICE) + h * HD + 4 * d4);
#pragma unroll
                for (int i = 0; i < 4; ++i) O[i] += f * part[i];
            }
        }
        float *dst = a.ws_acc + (((size_t)kvh * splits + split) * G + h) * HD + 4 * d4;
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[i] = O[i];
        if (d4 == 0) {
            a.ws_ml[(((size_t)kvh * splits + split) * G + h) * 2 + 0] = M;
            a.ws_ml[(((size_t)kvh * splits + split) * G + h) * 2 + 1] = L;
        }
    }
}

template <int HD, int G, bool FUSED, int NDIM, int LS, bool AGENT_OUT = false>
__device__ __forceinline__ void attn_decode_body(const AdArgs &a, float *sc, half_t *qs, half_t *knew, half_t *vnew,
                                                 float *s_m, float *s_l, int *s_last, const int pos,
                                                 const int n_active, const int split, const int d_begin,
                                                 const bool appender, const int kvh_arg = -1) {
    static_assert(LS == 256 || LS == 512, "span length");
    (void)s_m; // the statistics of a span live in ad_lds_ml; s_l and sc serve the merge of several spans below
    half_t *kst_all = ad_lds_kst<HD>();  // K blocks, one slice per wavefront
    float *ow_all = ad_lds_ow<NDIM, G>();  // unnormalised P.V per wavefront
    float *ml_all = ad_lds_ml<G>();      // (max, sum) per wavefront and head
    const int kvh = kvh_arg >= 0 ? kvh_arg : (int)blockIdx.x, splits = a.splits;
    const int tid = threadIdx.x;
    // one or two blocks per wavefront, each form with its own fixed number of loads in flight
    if (LS == 512 && pos + 1 - split * LS > 256)
        attn_decode_span<HD, G, FUSED, NDIM, LS, AGENT_OUT, LS / 256>(
            a, qs, knew, vnew, kst_all, ow_all, ml_all, pos, n_active, split, d_begin, appender, kvh);
    else
        attn_decode_span<HD, G, FUSED, NDIM, LS, AGENT_OUT, 1>(
            a, qs, knew, vnew, kst_all, ow_all, ml_all, pos, n_active, split, d_begin, appender, kvh);
    if (n_active == 1) return;

    // ---- 6. the last workgroup of this head merges the spans ------------------------------------
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        int old = atomicAdd(&a.counters[kvh], 1);
        *s_last = (old == n_active - 1);
    }
    __syncthreads();
    if (!*s_last) return;
    __threadfence();
    // (max, sum) of every span into LDS (reusing the score buffer) in one round of
    // independent loads, then per-span weights exp(m_s - M), then a weighted sum
    // whose loads do not depend on one another
    float *wgt = sc;                 // [n_active][G]: m_s, then the weights
    float *lsum = sc + n_active * G; // [n_active][G]: l_s
    for (int idx = tid; idx < n_active * G; idx += AD_THREADS) {
        const size_t b = ((size_t)kvh * splits + idx / G) * G + idx % G;
        wgt[idx] = a.ws_ml[b * 2];
        lsum[idx] = a.ws_ml[b * 2 + 1];
    }
    __syncthreads();
    if (tid < G) {
        float M = -FLT_MAX;
        for (int s = 0; s < n_active; ++s) M = fmaxf(M, wgt[s * G + tid]);
        float L = 0.f;
        for (int s = 0; s < n_active; ++s) {
            const float w = expf(wgt[s * G + tid] - M);
            wgt[s * G + tid] = w;
            L += lsum[s * G + tid] * w;
        }
        s_l[tid] = L;
    }
    __syncthreads();
    for (int idx = tid; idx < G * HD; idx += AD_THREADS) {
        const int h = idx / HD, d = idx % HD;
        float o = 0.f;
        int s = 0;
        for (; s + 8 <= n_active; s += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = a.ws_acc[(((size_t)kvh * splits + s + u) * G + h) * HD + d];
#pragma unroll
            for (int u = 0; u < 8; ++u) o += v[u] * wgt[(s + u) * G + h];
        }
        for (; s < n_active; ++s) o += a.ws_acc[(((size_t)kvh * splits + s) * G + h) * HD + d] * wgt[s * G + h];
        a.out[(size_t)(kvh * G + h) * HD + d] = (half_t)(o / s_l[h]);
    }
    if (tid == 0) a.counters[kvh] = 0; // ready for the next launch
}
