// Causal GQA attention for a block of query rows (prompt pass): streaming
// softmax over 64-key tiles on v_mfma_f32_32x32x16_f16; the [H,T,T] score
// tensor of the reference (src/inference/inference.cu:698-947) never exists.
//
// One workgroup = one KV head x 64 query rows (two 32-row tiles); each
// wavefront serves one query head on one tile, so the G heads of a group and
// both tiles share every K/V tile through LDS.
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

// Workgroup = one KV head x AP_QT query tiles (2, or 1 for groups of 8 heads); wavefront w serves query head
// kvh*G + w%G on tile w/G, so G*AP_QT wavefronts share every K/V tile.  K/V
// tiles are double buffered in LDS: tile kt+1 is requested from global memory
// into registers before the MFMAs of tile kt and written to the other buffer
// after them (one barrier per tile).
template <int HD, int G, int AP_QT>
__global__ __launch_bounds__(G *AP_QT * 64) void attn_prefill_kernel(const half_t *__restrict__ q, int ldq,
                                                                     const half_t *__restrict__ kc,
                                                                     const half_t *__restrict__ vc,
                                                                     half_t *__restrict__ out, int ldo, int T,
                                                                     int pos0, int max_pos) {
    constexpr int THREADS = G * AP_QT * 64;
    constexpr int KLD = HD + 8;       // K tile row stride (halves)
    constexpr int VLD = AP_BKEY + 8;  // V^T tile row stride
    constexpr int DS = HD / 16;       // k-steps of the first product
    constexpr int DT = HD / 32;       // 32-row tiles of O^T
    constexpr int KTILE = AP_BKEY * KLD, VTILE = HD * VLD;
    constexpr int KCH = AP_BKEY * HD / 8, VCH = HD * AP_BKEY / 8; // 16-byte chunks per tile
    constexpr int KL = (KCH + THREADS - 1) / THREADS, VL = (VCH + THREADS - 1) / THREADS;
    extern __shared__ __attribute__((aligned(16))) half_t smem[];
    half_t *Ks = smem;             // [2][KTILE]
    half_t *Vt = smem + 2 * KTILE; // [2][VTILE]

    const int n_qt = (T + AP_BQ - 1) / AP_BQ;
    // Workgroups are dispatched in the order of their linear id, x fastest.  KV head on x, row block on
    // y, longest rows first: the long workgroups of all heads start first and the short ones fill the
    // tail, and consecutive ids (which go round the XCDs) keep one KV head per XCD and its L2.
    const int blk = gridDim.y - 1 - blockIdx.y;
    const int kvh = blockIdx.x;
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int head = kvh * G + wave % G;
    int qtile = blk * AP_QT + wave / G;
    const bool live = qtile < n_qt; // a trailing wavefront without rows still helps with staging
    if (!live) qtile = n_qt - 1;
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

    const int my_last = (q0 + AP_BQ - 1 < T - 1 ? q0 + AP_BQ - 1 : T - 1) + pos0; // last key this wavefront sees
    int blk_last_q = (blk + 1) * AP_QT * AP_BQ - 1;
    if (blk_last_q > T - 1) blk_last_q = T - 1;
    const int n_tiles = (pos0 + blk_last_q) / AP_BKEY + 1;
    const half_t *kbase = kc + (size_t)kvh * max_pos * HD;
    const half_t *vbase = vc + (size_t)kvh * HD * max_pos;
    const float c2 = 1.44269504088896341f / sqrtf((float)HD); // log2(e) / sqrt(hd)
    const int pm = (n & ~0xC) | ((n & 8) >> 1) | ((n & 4) << 1); // pi(n)

    half8_t rk[KL], rv[VL];
    auto gload = [&](int key0) {
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const int c = tid + i * THREADS;
            if (KCH % THREADS == 0 || c < KCH) rk[i] = load8(kbase + (size_t)(key0 + c / (HD / 8)) * HD + (c % (HD / 8)) * 8);
        }
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const int c = tid + i * THREADS;
            if (VCH % THREADS == 0 || c < VCH)
                rv[i] = load8(vbase + (size_t)(c / (AP_BKEY / 8)) * max_pos + key0 + (c % (AP_BKEY / 8)) * 8);
        }
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const int c = tid + i * THREADS;
            if (KCH % THREADS == 0 || c < KCH) store8(Ks + buf * KTILE + (c / (HD / 8)) * KLD + (c % (HD / 8)) * 8, rk[i]);
        }
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const int c = tid + i * THREADS;
            if (VCH % THREADS == 0 || c < VCH)
                store8(Vt + buf * VTILE + (c / (AP_BKEY / 8)) * VLD + (c % (AP_BKEY / 8)) * 8, rv[i]);
        }
    };

    gload(0);
    sstore(0);
    // All loads issued so far (the query fragments among them) are complete from here on.  Without this
    // wait the compiler, which cannot tell the first pass of the loop from the others, makes every pass
    // wait for the query registers with counts that also drain the K/V prefetch issued at its top.
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    __syncthreads();
    for (int kt = 0; kt < n_tiles; ++kt) {
        const int key0 = kt * AP_BKEY;
        const int buf = kt & 1;
        if (kt + 1 < n_tiles) gload(key0 + AP_BKEY);
        if (live && key0 <= my_last) {
            const half_t *ks = Ks + buf * KTILE, *vt = Vt + buf * VTILE;
            // S^T for the two 32-key halves of the tile
            float16_t st[2];
#pragma unroll
            for (int kh = 0; kh < 2; ++kh) {
#pragma unroll
                for (int e = 0; e < 16; ++e) st[kh][e] = 0.f;
                const half_t *kr = ks + (32 * kh + pm) * KLD + 8 * hb;
#pragma unroll
                for (int s = 0; s < DS; ++s)
                    st[kh] = __builtin_amdgcn_mfma_f32_32x32x16_f16(load8(kr + 16 * s), qf[s], st[kh], 0, 0, 0);
            }
            // causal mask (only tiles that reach past the first row of this query tile need it) and
            // running max on the raw scores.  accumulator e of half kh is key
            // key0 + 32*kh + 16*(e/8) + 8*hb + e%8.  The softmax runs in base 2: with
            // c = log2(e)/sqrt(hd), p = 2^(s*c - m) is one fma and one v_exp_f32 per score; a masked
            // score (-FLT_MAX) gives 2^(-huge) = 0 without a select.
            float mx = -FLT_MAX;
            if (key0 + AP_BKEY - 1 > pos0 + q0) {
#pragma unroll
                for (int kh = 0; kh < 2; ++kh)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int key = key0 + 32 * kh + 16 * (e / 8) + 8 * hb + (e % 8);
                        const float sv = key <= qpos ? st[kh][e] : -FLT_MAX;
                        st[kh][e] = sv;
                        mx = fmaxf(mx, sv);
                    }
            } else {
#pragma unroll
                for (int kh = 0; kh < 2; ++kh)
#pragma unroll
                    for (int e = 0; e < 16; ++e) mx = fmaxf(mx, st[kh][e]);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run, mx * c2);
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            float psum = 0.f;
#pragma unroll
            for (int kh = 0; kh < 2; ++kh)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(st[kh][e], c2, -m_new));
                    st[kh][e] = p;
                    psum += p;
                }
            psum += __shfl_xor(psum, 32);
            l_run = l_run * alpha + psum;
            // the running max settles after the first tiles: skip the rescale of O^T when no lane needs it
            if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
#pragma unroll
                for (int t = 0; t < DT; ++t)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o[t][e] *= alpha;
            }
            m_run = m_new;

            // O^T += V^T . P^T, four 16-key steps
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                half8_t pb;
#pragma unroll
                for (int j = 0; j < 8; ++j) pb[j] = (half_t)st[u / 2][8 * (u % 2) + j];
#pragma unroll
                for (int t = 0; t < DT; ++t) {
                    half8_t vf = load8(vt + (32 * t + n) * VLD + 16 * u + 8 * hb);
                    o[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pb, o[t], 0, 0, 0);
                }
            }
        }
        if (kt + 1 < n_tiles) sstore(buf ^ 1);
        __syncthreads();
    }

    // O^T lane l: query q0 + l%32, dims 32t + 8*(e/4) + 4*(l/32) + e%4
    if (live && q0 + n < T) {
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
    constexpr int AP_QT = G >= 8 ? 1 : 2; // 32-row query tiles per workgroup (at most 8 wavefronts)
    const int n_qt = (T + AP_BQ - 1) / AP_BQ;
    dim3 grid(n_kv_heads, (n_qt + AP_QT - 1) / AP_QT);
    const size_t smem = sizeof(half_t) * 2 * ((size_t)AP_BKEY * (HD + 8) + (size_t)HD * (AP_BKEY + 8));
    auto kern = attn_prefill_kernel<HD, G, AP_QT>;
    static bool attr_set = false;
    if (!attr_set && smem > 48 * 1024) {
        LLM_HIP_CHECK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    kern<<<grid, dim3(G * AP_QT * 64), smem, s>>>(q, ldq, kc, vc, out, ldo, T, pos0, max_pos);
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
