// Causal GQA attention for one new token over the fp16 KV cache.
//
// Cache layout (per layer), chosen so that both passes stream contiguous
// memory per KV head:
//   K: [Hkv][max_pos][hd]   a position's hd values are contiguous  (scores = K . q)
//   V: [Hkv][hd][max_pos]   a dim's positions are contiguous       (out = V^T-rows . p)
//
// Grid (Hkv, splits): a workgroup owns one KV head and one span of positions
// and serves all G = Hq/Hkv query heads of the group, so each K/V byte is read
// once.  Per span: scores -> LDS, local max/sum, unnormalised P.V.  The last
// workgroup of a head to finish (a self-resetting counter) merges the spans.
// Scores, softmax and P.V stay in fp32 as in the reference
// (src/inference/inference.cu:736-947); only the final output is rounded.
#include <cfloat>
#include <cmath>

#include "common.hpp"

#define AD_THREADS 256
#define AD_MAX_SPLITS 256

struct AdShape {
    int splits;
    int ls_max; // longest span, multiple of 64
};

static AdShape ad_shape(int max_pos, int G) {
    AdShape s;
    s.splits = (max_pos + 255) / 256;
    if (s.splits < 1) s.splits = 1;
    if (s.splits > 32) s.splits = 32;
    for (;;) {
        int per = (max_pos + s.splits - 1) / s.splits;
        s.ls_max = (per + 63) / 64 * 64;
        if ((size_t)G * s.ls_max * sizeof(float) <= 40 * 1024 || s.splits >= AD_MAX_SPLITS) break;
        s.splits *= 2;
        if (s.splits > AD_MAX_SPLITS) s.splits = AD_MAX_SPLITS;
    }
    return s;
}

template <int HD, int G>
__global__ __launch_bounds__(AD_THREADS) void attn_decode_kernel(
    const half_t *__restrict__ q, const half_t *__restrict__ kc, const half_t *__restrict__ vc,
    half_t *__restrict__ out, int ctx_host, const int32_t *__restrict__ ctx_dev, int max_pos, int splits,
    int ls_max, float *__restrict__ ws_acc, float *__restrict__ ws_ml, int *__restrict__ counters) {
    constexpr int LPP = HD / 8;   // lanes per position in the score pass
    constexpr int PPW = 64 / LPP; // positions per wavefront pass
    extern __shared__ float sc[]; // [G][ls_max]
    __shared__ float s_m[G], s_l[G];
    __shared__ int s_last;

    const int kvh = blockIdx.x, split = blockIdx.y;
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    int ctx = ctx_host + (ctx_dev ? *ctx_dev : 0);
    if (ctx > max_pos) ctx = max_pos;
    if (ctx < 1) ctx = 1;
    const int per = (ctx + splits - 1) / splits;
    const int ls = (per + 63) / 64 * 64;
    const int n_active = (ctx + ls - 1) / ls;
    if (split >= n_active) return;
    const int s0 = split * ls;
    const int s1 = ctx < s0 + ls ? ctx : s0 + ls;
    const int len = s1 - s0;
    const int len_pad = (len + 63) / 64 * 64;

    // ---- scores ------------------------------------------------------------
    const int sub = lane % LPP;
    half8_t qreg[G];
#pragma unroll
    for (int h = 0; h < G; ++h) qreg[h] = load8(q + (size_t)(kvh * G + h) * HD + sub * 8);
    const float den = sqrtf((float)HD);
    const half_t *kbase = kc + (size_t)kvh * max_pos * HD;
    for (int j = s0 + wave * PPW + lane / LPP; j < s1; j += 4 * PPW) {
        half8_t kv = load8(kbase + (size_t)j * HD + sub * 8);
        float part[G];
#pragma unroll
        for (int h = 0; h < G; ++h) {
            part[h] = dot8(kv, qreg[h], 0.f);
#pragma unroll
            for (int off = LPP / 2; off >= 1; off >>= 1) part[h] += __shfl_xor(part[h], off);
        }
        if (sub == 0) {
#pragma unroll
            for (int h = 0; h < G; ++h) sc[h * ls_max + (j - s0)] = part[h] / den;
        }
    }
    __syncthreads();

    // ---- local softmax statistics: wavefront w takes heads w, w+4, ... -------
    for (int h = wave; h < G; h += 4) {
        float *row = sc + h * ls_max;
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

    // ---- unnormalised P.V: wavefront w takes dims [w*HD/4, (w+1)*HD/4) --------
    {
        const int rr = lane / 8, jc = lane % 8;
        const half_t *vbase = vc + (size_t)kvh * HD * max_pos + s0;
        for (int d0 = wave * (HD / 4); d0 < (wave + 1) * (HD / 4); d0 += 8) {
            const int d = d0 + rr;
            float acc[G];
#pragma unroll
            for (int h = 0; h < G; ++h) acc[h] = 0.f;
            for (int j = jc * 8; j < len; j += 64) {
                half8_t vv = load8(vbase + (size_t)d * max_pos + j);
                float vf[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) vf[i] = (j + i < len) ? (float)vv[i] : 0.f;
#pragma unroll
                for (int h = 0; h < G; ++h) {
                    const float *e = sc + h * ls_max + j;
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[h] = fmaf(e[i], vf[i], acc[h]);
                }
            }
#pragma unroll
            for (int h = 0; h < G; ++h) {
#pragma unroll
                for (int off = 4; off >= 1; off >>= 1) acc[h] += __shfl_xor(acc[h], off);
            }
            if (jc == 0) {
#pragma unroll
                for (int h = 0; h < G; ++h)
                    ws_acc[(((size_t)kvh * splits + split) * G + h) * HD + d] = acc[h];
            }
        }
    }
    if (tid < G) {
        ws_ml[(((size_t)kvh * splits + split) * G + tid) * 2 + 0] = s_m[tid];
        ws_ml[(((size_t)kvh * splits + split) * G + tid) * 2 + 1] = s_l[tid];
    }

    // ---- the last workgroup of this head merges the spans --------------------
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        int old = atomicAdd(&counters[kvh], 1);
        s_last = (old == n_active - 1);
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    for (int idx = tid; idx < G * HD; idx += AD_THREADS) {
        const int h = idx / HD, d = idx % HD;
        float M = -FLT_MAX;
        for (int s = 0; s < n_active; ++s)
            M = fmaxf(M, ws_ml[(((size_t)kvh * splits + s) * G + h) * 2]);
        float L = 0.f, o = 0.f;
        for (int s = 0; s < n_active; ++s) {
            const size_t b = ((size_t)kvh * splits + s) * G + h;
            const float wgt = expf(ws_ml[b * 2] - M);
            L += ws_ml[b * 2 + 1] * wgt;
            o += ws_acc[b * HD + d] * wgt;
        }
        out[(size_t)(kvh * G + h) * HD + d] = (half_t)(o / L);
    }
    if (tid == 0) counters[kvh] = 0; // ready for the next launch
}

template <int HD, int G>
static int launch_decode(const half_t *q, const half_t *kc, const half_t *vc, half_t *out, int ctx_host,
                         const int32_t *ctx_dev, int n_kv_heads, int max_pos, void *ws, hipStream_t s) {
    const AdShape sh = ad_shape(max_pos, G);
    const int Hq = n_kv_heads * G;
    float *ws_acc = (float *)ws;
    float *ws_ml = ws_acc + (size_t)Hq * AD_MAX_SPLITS * HD;
    int *counters = (int *)(ws_ml + (size_t)Hq * AD_MAX_SPLITS * 2);
    const size_t smem = (size_t)G * sh.ls_max * sizeof(float);
    LLM_REQUIRE(smem <= 64 * 1024, "llm_attn_decode: max_pos=%d needs %zu bytes of LDS", max_pos, smem);
    attn_decode_kernel<HD, G><<<dim3(n_kv_heads, sh.splits), dim3(AD_THREADS), smem, s>>>(
        q, kc, vc, out, ctx_host, ctx_dev, max_pos, sh.splits, sh.ls_max, ws_acc, ws_ml, counters);
    LLM_LAUNCH_CHECK("attn_decode_kernel");
    return LLM_OK;
}

extern "C" {

// Layout: acc [Hq][AD_MAX_SPLITS][hd] floats, (m,l) [Hq][AD_MAX_SPLITS][2]
// floats, then one int counter per KV head (<= Hq of them).  The counters must
// be zero before the first launch (llm_fill_zero the workspace once); every
// launch leaves them zero.
size_t llm_attn_decode_workspace_bytes(int n_heads, int head_dim) {
    return sizeof(float) * (size_t)n_heads * AD_MAX_SPLITS * (head_dim + 2) + sizeof(int) * (size_t)n_heads;
}

int llm_attn_decode(const uint16_t *q, const uint16_t *kc, const uint16_t *vc, uint16_t *out, int ctx_host,
                    const int32_t *ctx_dev, int n_heads, int n_kv_heads, int head_dim, int max_pos, void *workspace,
                    llm_stream_t stream) {
    LLM_REQUIRE(q && kc && vc && out && workspace, "llm_attn_decode: null pointer");
    LLM_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "llm_attn_decode: heads %d/%d", n_heads, n_kv_heads);
    LLM_REQUIRE(max_pos > 0 && max_pos % 64 == 0, "llm_attn_decode: max_pos=%d must be a multiple of 64", max_pos);
    LLM_REQUIRE(ctx_dev || (ctx_host >= 1 && ctx_host <= max_pos), "llm_attn_decode: ctx=%d of %d", ctx_host, max_pos);
    LLM_REQUIRE(aligned16(q) && aligned16(kc) && aligned16(vc), "llm_attn_decode: pointers must be 16-byte aligned");
    const int G = n_heads / n_kv_heads;
    hipStream_t s = (hipStream_t)stream;
    const half_t *qp = (const half_t *)q, *kp = (const half_t *)kc, *vp = (const half_t *)vc;
    half_t *op = (half_t *)out;
#define AD_CASE(HD_, G_)                                                                                   \
    if (head_dim == HD_ && G == G_)                                                                        \
        return launch_decode<HD_, G_>(qp, kp, vp, op, ctx_host, ctx_dev, n_kv_heads, max_pos, workspace, s);
    AD_CASE(128, 4)
    AD_CASE(128, 8)
    AD_CASE(128, 1)
    AD_CASE(64, 4)
    AD_CASE(64, 1)
    AD_CASE(32, 4)
    AD_CASE(32, 1)
#undef AD_CASE
    llm_set_error("llm_attn_decode: head_dim=%d with group size %d is not built", head_dim, G);
    return LLM_ERR_INVALID;
}

} // extern "C"
