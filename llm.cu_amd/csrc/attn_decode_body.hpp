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
    float *ws_acc, *ws_ml;
    int *counters;
};

// Every K and V load of the span is issued before anything else (a span is at
// most 512 positions: 16 + 16 loads of 16 bytes per thread at hd 128), so the
// whole span costs one trip to HBM instead of one per loop iteration.  In the
// fused form the new token's own K and V come from the projection row through
// LDS (and are written to the cache for later steps), so nothing waits on
// that write.
//
// NDIM is the number of head dims this workgroup produces, LS the span length.
// POLL_IN (with FUSED): a.q is a hand-over buffer that other workgroups of the same kernel are still
// filling: its words are read at device scope until none holds AD_EMPTY16 (the pattern the buffer was
// armed with, never written as a value) and staged in qkv_l ([(G + 2) * HD]: the group's queries, the new
// key, the new value).  The wait is bounded: after AD_POLL_LIMIT rounds *timeouts is incremented and the
// workgroup carries on.
#define AD_EMPTY16 0xFFFFu
#define AD_POLL_LIMIT (1 << 18)

template <int HD, int G, bool FUSED, int NDIM, int LS, bool TWOPASS = false, bool AGENT_OUT = false, bool POLL_IN = false>
__device__ __forceinline__ void attn_decode_body(const AdArgs &a, float *sc, half_t *qs, half_t *knew, half_t *vnew,
                                                 float *s_m, float *s_l, int *s_last, const int pos,
                                                 const int n_active, const int split, const int d_begin,
                                                 const bool appender, const int kvh_arg = -1, half_t *qkv_l = nullptr,
                                                 int *timeouts = nullptr) {
    constexpr int LPP = HD / 8;                    // lanes per position in the score pass
    constexpr int PPW = 64 / LPP;                  // positions per wavefront pass
    constexpr int KIT = LS / (AD_WAVES * PPW);  // K loads per thread
    constexpr int DPW = NDIM / AD_WAVES;           // dims per wavefront in the P.V pass
    static_assert(DPW >= 1, "too few dims for the workgroup");
    constexpr int RR = DPW < 8 ? DPW : 8;          // dim rows per pass
    constexpr int JL = 64 / RR;                    // lanes along positions (8, 16, 32 or 64)
    constexpr int VP = DPW / RR;                   // passes over dims
    constexpr int VIT = LS / (JL * 8);          // V loads per thread and pass
    constexpr int HALF = HD / 2;

    const int kvh = kvh_arg >= 0 ? kvh_arg : (int)blockIdx.x, splits = a.splits;
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int max_pos = a.max_pos;
    const int ctx = pos + 1;
    const int s0 = split * LS;
    const int len = ctx - s0 < LS ? ctx - s0 : LS;
    const int len_pad = (len + 63) / 64 * 64;
    half_t *kbase = a.kc + (size_t)kvh * max_pos * HD;
    half_t *vrow0 = a.vc + (size_t)kvh * HD * max_pos;
    const int lpos = pos - s0; // the new token inside this span (last span only)

    // ---- 1. all K and V loads of the span ----------------------------------------
    const int sub = lane % LPP;
    half8_t kreg[KIT];
#pragma unroll
    for (int it = 0; it < KIT; ++it) {
        const int j = it * (AD_WAVES * PPW) + wave * PPW + lane / LPP;
        kreg[it] = j < len ? load8(kbase + (size_t)(s0 + j) * HD + sub * 8) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
    const int rr = lane / JL, jc = lane % JL;
    half8_t vreg[VP][VIT];
#pragma unroll
    for (int p = 0; p < VP; ++p) {
        const int d = d_begin + wave * DPW + p * RR + rr;
#pragma unroll
        for (int it = 0; it < VIT; ++it) {
            const int j = (jc + JL * it) * 8;
            vreg[p][it] = j < len ? load8(vrow0 + (size_t)d * max_pos + s0 + j) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }

    // ---- 2. queries into LDS; fused: rotate them and the new K, append K/V ---------
    if (FUSED) {
        const int Hq = a.n_kv_heads * G;
        const half_t *qkv = a.q;
        const float *cs = a.table + (size_t)pos * HALF * 2;
        if (POLL_IN) {
            constexpr int NQ = G * HD / 2, NK = HD / 2; // 32-bit words
            const uint32_t *base = reinterpret_cast<const uint32_t *>(qkv);
            int spins = 0;
            for (int wi = tid; wi < NQ + 2 * NK; wi += AD_THREADS) {
                const size_t sw = wi < NQ        ? (size_t)kvh * G * HD / 2 + wi
                                  : wi < NQ + NK ? ((size_t)Hq * HD + (size_t)kvh * HD) / 2 + (wi - NQ)
                                                 : ((size_t)(Hq + a.n_kv_heads) * HD + (size_t)kvh * HD) / 2 + (wi - NQ - NK);
                uint32_t v;
                for (;;) {
                    v = __hip_atomic_load(base + sw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if ((v & 0xFFFFu) != AD_EMPTY16 && (v >> 16) != AD_EMPTY16) break;
                    if (++spins > AD_POLL_LIMIT) {
                        if (timeouts) atomicAdd(timeouts, 1);
                        break;
                    }
                    __builtin_amdgcn_s_sleep(8); // a few hundred cycles: the pollers must not crowd the producers' memory traffic
                }
                reinterpret_cast<uint32_t *>(qkv_l)[wi] = v;
            }
            __syncthreads();
        }
        for (int p = tid; p < (G + 1) * HALF; p += AD_THREADS) {
            const int h = p / HALF, i = p % HALF; // h == G: the new key
            const half_t *src = POLL_IN ? qkv_l + (size_t)h * HD + 2 * i
                                : h < G ? qkv + (size_t)(kvh * G + h) * HD + 2 * i
                                        : qkv + (size_t)Hq * HD + (size_t)kvh * HD + 2 * i;
            const float c = cs[2 * i], sn = cs[2 * i + 1];
            const float e = (float)src[0], o = (float)src[1];
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
        const half_t *vsrc = POLL_IN ? qkv_l + (size_t)(G + 1) * HD : qkv + (size_t)(Hq + a.n_kv_heads) * HD + (size_t)kvh * HD;
        for (int d = tid; d < HD; d += AD_THREADS) {
            const half_t v = vsrc[d];
            vnew[d] = v;
            if (appender) vrow0[(size_t)d * max_pos + pos] = v;
        }
    } else {
        for (int c = tid * 8; c < G * HD; c += AD_THREADS * 8) store8(qs + c, load8(a.q + (size_t)kvh * G * HD + c));
    }
    __syncthreads();

    // ---- 3. scores ---------------------------------------------------------------------
    // On the matrix pipe: a block of 16 positions (NPB passes of this wavefront) against the G heads as columns
    // 0..G-1 of a 16-column operand.  The K registers keep their row-contiguous load pattern (whole 256-byte rows
    // per position); a wavefront turns a block into the MFMA's row operand through its own slice of LDS, with
    // no workgroup barrier.  Lane (mg, mn) of the result holds rows 4 mg .. + 3 of the block for head mn.
    {
        constexpr int KS = HD / 32;   // k-steps of 32 dims
        constexpr int NPB = 16 / PPW; // passes per block of 16 positions
        constexpr int KLD = HD + 8;   // row stride of the staging slice (halves): fragment reads without bank conflicts
        static_assert(KIT % NPB == 0 && G <= 16, "score blocks");
        __shared__ __attribute__((aligned(16))) half_t kst_all[AD_WAVES * 16 * KLD];
        half_t *kst = kst_all + wave * 16 * KLD;
        const int mg = lane / 16, mn = lane % 16;
        half8_t qreg[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            qreg[ks] = mn < G ? load8(qs + mn * HD + 32 * ks + 8 * mg) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        const float scale = 1.0f / sqrtf((float)HD);
#pragma unroll
        for (int b = 0; b < KIT / NPB; ++b) {
            const int it0 = b * NPB;
            if (it0 * (AD_WAVES * PPW) + wave * PPW < len) { // wave-uniform: skip blocks beyond the span
#pragma unroll
                for (int q = 0; q < NPB; ++q) {
                    const int j = (it0 + q) * (AD_WAVES * PPW) + wave * PPW + lane / LPP;
                    half8_t kv = kreg[it0 + q];
                    if (FUSED && j == lpos) kv = load8(knew + sub * 8);
                    store8(kst + (q * PPW + lane / LPP) * KLD + sub * 8, kv);
                }
                float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(load8(kst + mn * KLD + 32 * ks + 8 * mg), qreg[ks], acc, 0, 0, 0);
                if (mn < G) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int m = 4 * mg + i; // row of the block: pass m / PPW, position m % PPW of that pass
                        const int j = (it0 + m / PPW) * (AD_WAVES * PPW) + wave * PPW + m % PPW;
                        if (j < len) sc[mn * LS + j] = acc[i] * scale;
                    }
                }
            }
        }
    }
    __syncthreads();

    // ---- 4. local softmax statistics: wavefront w takes heads w, w+8, ... ------------------
    for (int h = wave; h < G; h += AD_WAVES) {
        float *row = sc + h * LS;
        float mx = -FLT_MAX;
        for (int j = lane; j < len; j += 64) mx = fmaxf(mx, row[j]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int j = lane; j < len_pad; j += 64) {
            float e = j < len ? expf(row[j] - mx) : 0.f;
            row[j] = e;
            sum += e;
        }
        sum = wave_sum(sum);
        if (lane == 0) {
            s_m[h] = mx;
            s_l[h] = sum;
        }
    }
    __syncthreads();

    // ---- 5. unnormalised P.V from the registers ----------------------------------------------
#pragma unroll
    for (int p = 0; p < VP; ++p) {
        const int d = d_begin + wave * DPW + p * RR + rr;
        float acc[G];
#pragma unroll
        for (int h = 0; h < G; ++h) acc[h] = 0.f;
#pragma unroll
        for (int it = 0; it < VIT; ++it) {
            const int j = (jc + JL * it) * 8;
            if (j < len) {
                float vf[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) vf[i] = (float)vreg[p][it][i];
                if (FUSED && lpos >= j && lpos < j + 8) { // the chunk that holds the new token (rare)
                    const float vn = (float)vnew[d];
#pragma unroll
                    for (int i = 0; i < 8; ++i) vf[i] = (j + i == lpos) ? vn : vf[i];
                }
                if (j + 8 > len) { // the chunk that straddles the end of the span (rare)
#pragma unroll
                    for (int i = 0; i < 8; ++i) vf[i] = (j + i < len) ? vf[i] : 0.f;
                }
#pragma unroll
                for (int h = 0; h < G; ++h) {
                    const float *e = sc + h * LS + j;
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[h] = fmaf(e[i], vf[i], acc[h]);
                }
            }
        }
#pragma unroll
        for (int h = 0; h < G; ++h) {
            if (JL <= 16) {
                acc[h] = group_sum<(JL <= 16 ? JL : 16)>(acc[h]);
            } else {
                acc[h] = group_sum<16>(acc[h]);
                acc[h] += __shfl_xor(acc[h], 16);
                if (JL == 64) acc[h] += __shfl_xor(acc[h], 32);
            }
        }
        if (jc == 0) {
            if (n_active == 1 && !TWOPASS) {
#pragma unroll
                for (int h = 0; h < G; ++h) {
                    const half_t r = (half_t)(acc[h] / s_l[h]);
                    if (AGENT_OUT) { // collected in LDS (the queries are no longer needed), stored wide below
                        uint16_t bits = __builtin_bit_cast(uint16_t, r);
                        if (bits == 0xFFFFu) bits = 0xFFFEu; // 0xFFFF marks "not written yet" for the reader
                        reinterpret_cast<uint16_t *>(qs)[h * NDIM + (d - d_begin)] = bits;
                    }
                    else
                        a.out[(size_t)(kvh * G + h) * HD + d] = r;
                }
            } else {
#pragma unroll
                for (int h = 0; h < G; ++h) a.ws_acc[(((size_t)kvh * splits + split) * G + h) * HD + d] = acc[h];
            }
        }
    }
    if (AGENT_OUT) {
        // This workgroup's G x NDIM results go out as 8-byte device-scope stores (written through to the
        // point where every XCD reads them): 2-byte write-through stores cost a read-modify-write each.
        static_assert(!AGENT_OUT || NDIM % 4 == 0, "results are stored four at a time");
        __syncthreads();
        if (tid < G * NDIM / 4) {
            const int h = tid / (NDIM / 4), q = tid % (NDIM / 4);
            const unsigned long long v = reinterpret_cast<const unsigned long long *>(qs)[tid];
            __hip_atomic_store(reinterpret_cast<unsigned long long *>(a.out + (size_t)(kvh * G + h) * HD + d_begin) + q, v,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (n_active == 1 && !TWOPASS) return;
    if (tid < G) {
        a.ws_ml[(((size_t)kvh * splits + split) * G + tid) * 2 + 0] = s_m[tid];
        a.ws_ml[(((size_t)kvh * splits + split) * G + tid) * 2 + 1] = s_l[tid];
    }

    if (TWOPASS) return; // attn_merge_kernel combines the spans

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
