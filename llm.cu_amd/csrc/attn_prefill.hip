// Causal GQA attention for a block of query rows (prompt pass): streaming
// softmax over 64-key tiles on v_mfma_f32_32x32x16_f16; the [H,T,T] score
// tensor of the reference (src/inference/inference.cu:698-947) never exists.
//
// One workgroup = one KV head x 32 query rows; wavefront w serves query head
// kvh*G + w, so the G heads of a group share every K/V tile through LDS.
//
// The kernel computes the transposed problem so that no register shuffles are
// needed between the two matrix products:
//   S^T[key, q]  = K[key, :] . Q[q, :]          A = K rows,   B = Q rows
//   O^T[d,   q] += V^T[d, key] . P^T[key, q]    A = V^T rows, B = P^T
// A 32x32 MFMA result holds, in lane l, column q = l%32 and rows
// 8*(i/4) + 4*(l/32) + i%4 (i < 16); the B operand of the next product wants,
// in the same lane, 8 consecutive k-slots 8*(l/32) + j.  Loading the K rows
// of the first product in the order pi(m) = m with bits 2 and 3 swapped makes
// accumulators 8u..8u+7 exactly the keys 16u + 8*(l/32) + 0..7 of the tile,
// i.e. already the B fragment (after fp16 packing).  V is cached transposed
// ([Hkv][hd][max_pos]), so the A fragment of the second product is one
// 16-byte LDS read.
//
// Softmax statistics are per query = per lane column, so rescaling O^T is a
// per-lane multiply.  P is rounded to fp16 for the MFMA (the reference keeps
// P in fp32; the difference is below the fp16 rounding of the output).
#include <cfloat>
#include <cmath>

#include "common.hpp"

#define AP_BQ 32
#define AP_BKEY 64

template <int HD, int G>
__global__ __launch_bounds__(G * 64) void attn_prefill_kernel(const half_t *__restrict__ q, int ldq,
                                                              const half_t *__restrict__ kc,
                                                              const half_t *__restrict__ vc,
                                                              half_t *__restrict__ out, int ldo, int T,
                                                              int pos0, int max_pos) {
    constexpr int THREADS = G * 64;
    constexpr int KLD = HD + 8;       // K tile row stride (halves)
    constexpr int VLD = AP_BKEY + 8;  // V^T tile row stride
    constexpr int DS = HD / 16;       // k-steps of the first product
    constexpr int DT = HD / 32;       // 32-row tiles of O^T
    __shared__ __attribute__((aligned(16))) half_t Ks[AP_BKEY * KLD];
    __shared__ __attribute__((aligned(16))) half_t Vt[HD * VLD];

    const int qtile = gridDim.x - 1 - blockIdx.x; // longest rows first
    const int kvh = blockIdx.y;
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int head = kvh * G + wave;
    const int n = lane % 32, hb = lane / 32;
    const int q0 = qtile * AP_BQ;
    const int qrow = q0 + n < T ? q0 + n : T - 1;
    const int qpos = pos0 + q0 + n; // absolute position of this lane's query

    half8_t qf[DS];
#pragma unroll
    for (int s = 0; s < DS; ++s) qf[s] = load8(q + (size_t)qrow * ldq + (size_t)head * HD + 16 * s + 8 * hb);

    float16_t o[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
    float m_run = -FLT_MAX, l_run = 0.f;

    const int last_q = q0 + AP_BQ - 1 < T - 1 ? q0 + AP_BQ - 1 : T - 1;
    const int kmax = pos0 + last_q; // last key any row of this tile may see
    const int n_tiles = kmax / AP_BKEY + 1;
    const half_t *kbase = kc + (size_t)kvh * max_pos * HD;
    const half_t *vbase = vc + (size_t)kvh * HD * max_pos;
    const float scale = 1.0f / sqrtf((float)HD);
    const int pm = (n & ~0xC) | ((n & 8) >> 1) | ((n & 4) << 1); // pi(n)

    for (int kt = 0; kt < n_tiles; ++kt) {
        const int key0 = kt * AP_BKEY;
        __syncthreads(); // previous tile fully consumed
        for (int i = tid; i < AP_BKEY * HD / 8; i += THREADS) {
            const int r = i / (HD / 8), c = (i % (HD / 8)) * 8;
            store8(Ks + r * KLD + c, load8(kbase + (size_t)(key0 + r) * HD + c));
        }
        for (int i = tid; i < HD * AP_BKEY / 8; i += THREADS) {
            const int d = i / (AP_BKEY / 8), c = (i % (AP_BKEY / 8)) * 8;
            store8(Vt + d * VLD + c, load8(vbase + (size_t)d * max_pos + key0 + c));
        }
        __syncthreads();

        // S^T for the two 32-key halves of the tile
        float16_t st[2];
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) {
#pragma unroll
            for (int e = 0; e < 16; ++e) st[kh][e] = 0.f;
            const half_t *kr = Ks + (32 * kh + pm) * KLD + 8 * hb;
#pragma unroll
            for (int s = 0; s < DS; ++s)
                st[kh] = __builtin_amdgcn_mfma_f32_32x32x16_f16(load8(kr + 16 * s), qf[s], st[kh], 0, 0, 0);
        }
        // scale, causal mask, running max.  accumulator e of half kh is key
        // key0 + 32*kh + 16*(e/8) + 8*hb + e%8.
        float mx = -FLT_MAX;
#pragma unroll
        for (int kh = 0; kh < 2; ++kh)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int key = key0 + 32 * kh + 16 * (e / 8) + 8 * hb + (e % 8);
                float s = st[kh][e] * scale;
                s = key <= qpos ? s : -FLT_MAX;
                st[kh][e] = s;
                mx = fmaxf(mx, s);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        const float alpha = __expf(m_run - m_new);
        float psum = 0.f;
#pragma unroll
        for (int kh = 0; kh < 2; ++kh)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float s = st[kh][e];
                const float p = s == -FLT_MAX ? 0.f : __expf(s - m_new);
                st[kh][e] = p;
                psum += p;
            }
        psum += __shfl_xor(psum, 32);
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[t][e] *= alpha;

        // O^T += V^T . P^T, four 16-key steps
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            half8_t pb;
#pragma unroll
            for (int j = 0; j < 8; ++j) pb[j] = (half_t)st[u / 2][8 * (u % 2) + j];
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                half8_t vf = load8(Vt + (32 * t + n) * VLD + 16 * u + 8 * hb);
                o[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pb, o[t], 0, 0, 0);
            }
        }
    }

    // O^T lane l: query q0 + l%32, dims 32t + 8*(e/4) + 4*(l/32) + e%4
    if (q0 + n < T) {
        const float inv = 1.0f / l_run;
        half_t *orow = out + (size_t)(q0 + n) * ldo + (size_t)head * HD;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                half4_t v;
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = (half_t)(o[t][4 * e4 + i] * inv);
                *reinterpret_cast<half4_t *>(orow + 32 * t + 8 * e4 + 4 * hb) = v;
            }
    }
}

template <int HD, int G>
static int launch_prefill(const half_t *q, int ldq, const half_t *kc, const half_t *vc, half_t *out, int ldo,
                          int T, int pos0, int n_kv_heads, int max_pos, hipStream_t s) {
    dim3 grid((T + AP_BQ - 1) / AP_BQ, n_kv_heads);
    attn_prefill_kernel<HD, G><<<grid, dim3(G * 64), 0, s>>>(q, ldq, kc, vc, out, ldo, T, pos0, max_pos);
    LLM_LAUNCH_CHECK("attn_prefill_kernel");
    return LLM_OK;
}

extern "C" int llm_attn_prefill(const uint16_t *q, int ldq, const uint16_t *kc, const uint16_t *vc,
                                uint16_t *out, int ldo, int T, int pos0, int n_heads, int n_kv_heads,
                                int head_dim, int max_pos, llm_stream_t stream) {
    LLM_REQUIRE(q && kc && vc && out, "llm_attn_prefill: null pointer");
    LLM_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "llm_attn_prefill: heads %d/%d", n_heads, n_kv_heads);
    LLM_REQUIRE(T >= 0 && pos0 >= 0 && pos0 + T <= max_pos, "llm_attn_prefill: rows %d..%d of %d", pos0, pos0 + T,
                max_pos);
    LLM_REQUIRE(max_pos % 64 == 0, "llm_attn_prefill: max_pos=%d must be a multiple of 64", max_pos);
    LLM_REQUIRE(ldq % 8 == 0 && ldq >= n_heads * head_dim && ldo % 4 == 0 && ldo >= n_heads * head_dim,
                "llm_attn_prefill: ldq=%d ldo=%d", ldq, ldo);
    LLM_REQUIRE(aligned16(q) && aligned16(kc) && aligned16(vc) && ((uintptr_t)out & 7u) == 0,
                "llm_attn_prefill: pointers must be 16-byte aligned");
    if (T == 0) return LLM_OK;
    const int G = n_heads / n_kv_heads;
    hipStream_t s = (hipStream_t)stream;
    const half_t *qp = (const half_t *)q, *kp = (const half_t *)kc, *vp = (const half_t *)vc;
    half_t *op = (half_t *)out;
#define AP_CASE(HD_, G_)                                                                        \
    if (head_dim == HD_ && G == G_)                                                             \
        return launch_prefill<HD_, G_>(qp, ldq, kp, vp, op, ldo, T, pos0, n_kv_heads, max_pos, s);
    AP_CASE(128, 4)
    AP_CASE(128, 8)
    AP_CASE(128, 1)
    AP_CASE(64, 4)
    AP_CASE(64, 1)
    AP_CASE(32, 4)
    AP_CASE(32, 1)
#undef AP_CASE
    llm_set_error("llm_attn_prefill: head_dim=%d with group size %d is not built", head_dim, G);
    return LLM_ERR_INVALID;
}
