// Causal GQA attention for a block of query rows (prompt pass): streaming
// softmax over key tiles on v_mfma_f32_32x32x16_f16; the [H,T,T] score
// tensor of the reference (src/inference/inference.cu:698-947) never exists.
//
// Two kernels share the arithmetic.  attn_prefill_kernel (any supported head
// size and group) is described next; attn_prefill_pipe_kernel (head size 128,
// four query heads per KV head, the LLaMA3-8B shape) is the software-pipelined
// form further down.
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
#include <type_traits>

#include "common.hpp"

#define AP_BQ 32
#define AP_BKEY 64
#define AP_PIPE_MIN_ROWS 64 // shorter blocks of rows take attn_prefill_kernel

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
    auto gload_k = [&](int key0) {
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const int c = tid + i * THREADS;
            if (KCH % THREADS == 0 || c < KCH) rk[i] = load8(kbase + (size_t)(key0 + c / (HD / 8)) * HD + (c % (HD / 8)) * 8);
        }
    };
    auto gload_v = [&](int key0) {
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const int c = tid + i * THREADS;
            if (VCH % THREADS == 0 || c < VCH)
                rv[i] = load8(vbase + (size_t)(c / (AP_BKEY / 8)) * max_pos + key0 + (c % (AP_BKEY / 8)) * 8);
        }
    };
    auto sstore_k = [&](int buf) {
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const int c = tid + i * THREADS;
            if (KCH % THREADS == 0 || c < KCH) store8(Ks + buf * KTILE + (c / (HD / 8)) * KLD + (c % (HD / 8)) * 8, rk[i]);
        }
    };
    auto sstore_v = [&](int buf) {
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const int c = tid + i * THREADS;
            if (VCH % THREADS == 0 || c < VCH)
                store8(Vt + buf * VTILE + (c / (AP_BKEY / 8)) * VLD + (c % (AP_BKEY / 8)) * 8, rv[i]);
        }
    };

    // The two matrix products of a tile, with pinned instruction order (a scheduling fence after every
    // MFMA): accumulators alternate, so no MFMA waits for the one before it, and the LDS fragment of MFMA
    // i + LA is read behind MFMA i.  Left alone the scheduler reads each fragment right in front of its
    // MFMA and both wavefronts of a SIMD sit out the LDS latency together.
    constexpr int NQ = 2 * DS, NP = 4 * DT, LA = 4; // MFMAs per product; read-ahead
    auto kfrag = [&](const half_t *ks, int i) { return load8(ks + (32 * (i % 2) + pm) * KLD + 8 * hb + 16 * (i / 2)); };
    auto vfrag = [&](const half_t *vt, int i) { return load8(vt + (32 * (i % DT) + n) * VLD + 16 * (i / DT) + 8 * hb); };
    // lanes l and l ^ 32 hold the two halves of a query's keys
    auto xhalf = [&](float x, float &lo, float &hi) {
        auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
        lo = __uint_as_float(r[0]);
        hi = __uint_as_float(r[1]);
    };

    // Softmax of one tile in slices, so that it can run between the MFMAs of the next tile's first product.
    // The state of the tile in flight lives in these variables; slice i of NQ:
    //   [0, NQ/4)   running max over the 32 raw scores of the lane
    //   NQ/4        other half of the keys; new running max m_new, rescale factor alpha
    //   [NQ/2, NQ)  p = 2^(s*c2 - m_new), partial row sum
    // sm_finish adds the row sum into l_run and rescales O^T if some lane's max moved.  The softmax runs in
    // base 2: with c2 = log2(e)/sqrt(hd), p is one fma and one v_exp_f32 per score.
    float sm_mx = -FLT_MAX, sm_new = 0.f, sm_alpha = 1.f, sm_sum = 0.f;
    half2_t pk[16]; // the 32 probabilities of the tile whose softmax ran last, as fp16 pairs
    auto sm_slice = [&](float16_t (&st)[2], int i) {
        constexpr int PM = 128 / NQ, PE = 64 / NQ; // scores per max slice / per exp slice
        if (i < NQ / 4) {
            if (i == 0) sm_mx = -FLT_MAX;
#pragma unroll
            for (int j = 0; j < PM; ++j) {
                const int e = i * PM + j;
                sm_mx = fmaxf(sm_mx, st[e / 16][e % 16]);
            }
        }
        if (i == NQ / 4) {
            float lo, hi;
            xhalf(sm_mx, lo, hi);
            sm_new = fmaxf(m_run, fmaxf(lo, hi) * c2);
            sm_alpha = __builtin_amdgcn_exp2f(m_run - sm_new);
            sm_sum = 0.f;
        }
        if (i >= NQ / 2) {
            // probabilities are rounded to fp16 here (the second product takes them in fp16) and the row sum
            // is taken over the rounded values, two per v_dot2_f32_f16: numerator and denominator of the
            // output then use the same weights, and the sum costs half the instructions
            static_assert(PE % 2 == 0, "pairs");
#pragma unroll
            for (int j = 0; j < PE; j += 2) {
                const int e = (i - NQ / 2) * PE + j;
                const float p0 = __builtin_amdgcn_exp2f(fmaf(st[e / 16][e % 16], c2, -sm_new));
                const float p1 = __builtin_amdgcn_exp2f(fmaf(st[(e + 1) / 16][(e + 1) % 16], c2, -sm_new));
                const half2_t h = {(half_t)p0, (half_t)p1};
                pk[e / 2] = h;
                sm_sum = __builtin_amdgcn_fdot2(h, half2_t{(half_t)1.0f, (half_t)1.0f}, sm_sum, false);
            }
        }
    };
    auto sm_finish = [&]() {
        float lo, hi;
        xhalf(sm_sum, lo, hi);
        l_run = l_run * sm_alpha + (lo + hi);
        // the running max settles after the first tiles: skip the rescale of O^T when no lane needs it
        if (__builtin_amdgcn_ballot_w64(sm_new != m_run) != 0) {
#pragma unroll
            for (int t = 0; t < DT; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[t][e] *= sm_alpha;
        }
        m_run = sm_new;
    };
    // causal mask of a tile that reaches past the first row of this query tile: accumulator e of half kh is
    // key key0 + 32*kh + 16*(e/8) + 8*hb + e%8; a masked score (-FLT_MAX) gives 2^(-huge) = 0
    auto mask = [&](float16_t (&st)[2], int key0) {
        if (key0 + AP_BKEY - 1 > pos0 + q0) {
#pragma unroll
            for (int kh = 0; kh < 2; ++kh)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = key0 + 32 * kh + 16 * (e / 8) + 8 * hb + (e % 8);
                    st[kh][e] = key <= qpos ? st[kh][e] : -FLT_MAX;
                }
        }
    };
    // first product of tile kt into st, optionally with the softmax of the previous tile (in prev) between
    // its MFMAs; the first V fragments of the tile whose second product follows (in vt) ride on its last MFMAs
    half8_t vf[LA];
    auto qk = [&](float16_t (&st)[2], int kt, auto with_softmax, float16_t (&prev)[2], const half_t *vt) {
        const half_t *ks = Ks + (kt & 1) * KTILE;
#pragma unroll
        for (int e = 0; e < 16; ++e) st[0][e] = st[1][e] = 0.f;
        half8_t kf[LA];
#pragma unroll
        for (int j = 0; j < LA; ++j)
            if (j < NQ) kf[j] = kfrag(ks, j);
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            st[i % 2] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[i % LA], qf[i / 2], st[i % 2], 0, 0, 0);
            if (i + LA < NQ) kf[i % LA] = kfrag(ks, i + LA);
            else if (vt && i + LA - NQ < LA && i + LA - NQ < NP) vf[i + LA - NQ] = vfrag(vt, i + LA - NQ);
            if (decltype(with_softmax)::value) sm_slice(prev, i);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // second product: O^T += V^T . P^T with P = st (fp16), V tile in vt; vf[0..LA) already hold its first fragments
    auto pv = [&](float16_t (&st)[2], const half_t *vt) {
        half8_t pb;
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            if (i % DT == 0) {
                const int u = i / DT;
#pragma unroll
                for (int j = 0; j < 8; ++j) pb[j] = pk[(u / 2) * 8 + 4 * (u % 2) + j / 2][j % 2];
            }
            o[i % DT] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[i % LA], pb, o[i % DT], 0, 0, 0);
            if (i + LA < NP) vf[i % LA] = vfrag(vt, i + LA);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto load_vf = [&](const half_t *vt) {
#pragma unroll
        for (int j = 0; j < LA; ++j)
            if (j < NP) vf[j] = vfrag(vt, j);
    };

    // Schedule.  K runs two tiles ahead of the tile being finished, V one: step t finishes tile t (softmax,
    // second product) while the first product of tile t + 1 is computed between the softmax instructions,
    // so the matrix pipe works under the softmax.  The last two tiles of the workgroup are the only ones
    // that can need the causal mask or lie beyond a wavefront's rows; they take the plain path below.
    //   LDS: K tile t in Ks[t & 1], V tile t in Vt[t & 1]; step t stores K(t + 2) and V(t + 1) at its end.
    gload_k(0);
    gload_v(0);
    sstore_k(0);
    sstore_v(0);
    if (n_tiles > 1) {
        gload_k(AP_BKEY);
        sstore_k(1);
    }
    // All loads issued so far (the query fragments among them) are complete from here on.  Without this
    // wait the compiler, which cannot tell the first pass of a loop from the others, makes every pass
    // wait for the query registers with counts that also drain the K/V prefetch issued at its top.
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    __syncthreads();

    const int n_main = n_tiles > 2 ? n_tiles - 2 : 0;
    float16_t sa[2], sb[2];
    auto stage_in = [&](int kt) { // global loads of the tiles that step kt stores
        if (kt + 2 < n_tiles) gload_k((kt + 2) * AP_BKEY);
        if (kt + 1 < n_tiles) gload_v((kt + 1) * AP_BKEY);
    };
    auto stage_out = [&](int kt) {
        if (kt + 2 < n_tiles) sstore_k(kt & 1);
        if (kt + 1 < n_tiles) sstore_v((kt + 1) & 1);
        __syncthreads();
    };
    // main step on tile kt < n_main: scores of tile kt are in cur, those of tile kt + 1 go to nxt
    auto step = [&](int kt, float16_t (&cur)[2], float16_t (&nxt)[2]) {
        stage_in(kt);
        if (live) {
            const half_t *vt = Vt + (kt & 1) * VTILE;
            qk(nxt, kt + 1, std::true_type{}, cur, vt);
            sm_finish();
            pv(cur, vt);
        }
        stage_out(kt);
    };
    if (live) qk(sa, 0, std::false_type{}, sa, (const half_t *)nullptr);
    int kt = 0;
    for (; kt + 1 < n_main; kt += 2) {
        step(kt, sa, sb);
        step(kt + 1, sb, sa);
    }
    if (kt < n_main) {
        step(kt, sa, sb);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            sa[0][e] = sb[0][e];
            sa[1][e] = sb[1][e];
        }
        ++kt;
    }
    // plain path: tile kt has its scores in sa; the tile after it (if any) is computed here
    for (; kt < n_tiles; ++kt) {
        const int key0 = kt * AP_BKEY;
        stage_in(kt);
        if (live && key0 <= my_last) {
            const half_t *vt = Vt + (kt & 1) * VTILE;
            load_vf(vt);
            mask(sa, key0);
#pragma unroll
            for (int i = 0; i < NQ; ++i) sm_slice(sa, i);
            sm_finish();
            pv(sa, vt);
        }
        if (kt + 1 < n_tiles && live && key0 + AP_BKEY <= my_last) qk(sa, kt + 1, std::false_type{}, sa, (const half_t *)nullptr);
        stage_out(kt);
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

#define AP_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

// ---- software-pipelined form for head size 128 and four query heads per KV head -----------------------------
//
// Same workgroup shape (one KV head x 64 query rows, wavefront = one head x 32 rows, two wavefronts per SIMD) and
// the same two transposed products, organised around what bounds the kernel on this part: board power.  Time
// follows the energy of the instructions issued, so the kernel issues fewer of them:
//  * The unit of work is a chunk of 32 keys.  One iteration computes the scores of chunk c + 1 (8 MFMAs), the
//    probabilities of chunk c (16 values per lane) and O^T += V^T . P^T of chunk c - 1 (8 MFMAs); the softmax
//    instructions sit between the MFMAs (a SIMD takes about four vector instructions under each MFMA), two
//    score and two probability sets alternate, and two iterations form one trip of the loop.
//  * K and V^T tiles of 64 keys travel from global memory straight into a ring of four LDS stages
//    (buffer_load ... lds, no staging registers, no LDS stores); a lane fetches the 16-byte chunk that the
//    bank swizzle assigns to its LDS slot.  One workgroup barrier per tile.
//  * The softmax keeps a reference maximum per query that moves only when a probability would leave the fp16
//    range (then the row sum reads infinite): the running maximum is not computed per chunk, and O^T is
//    rescaled a handful of times per query instead of whenever any lane's maximum moves.  Probabilities are
//    2^(s c - m_ref) <= 65504 in fp16, sums and O^T in fp32, so the result is the same softmax: O^T / l.
typedef uint32_t ap_u4_t __attribute__((ext_vector_type(4)));
typedef uint32_t ap_u8_t __attribute__((ext_vector_type(8)));

template <int G, bool ROPE_Q>
__global__ __launch_bounds__(G * 128, 1) void attn_prefill_pipe_kernel(const half_t *__restrict__ q, int ldq,
                                                                       const half_t *__restrict__ kc,
                                                                       const half_t *__restrict__ vc,
                                                                       half_t *__restrict__ out, int ldo, int T,
                                                                       int pos0, int max_pos,
                                                                       const float *__restrict__ table) {
    // ROPE_Q: q holds the projection as stored; every wavefront rotates its own query fragments by the angles of their
    // positions (table: [max_pos][64][2], as llm_rope uses it) right after loading them -- the arithmetic of the
    // RoPE kernel on the same elements, so the same bits, without a pass over Q in memory.
    static_assert(G == 4, "eight wavefronts, two per SIMD");
    constexpr int HD = 128, NW = 2 * G, THREADS = NW * 64;
    constexpr int LPT = 32 / NW;            // tile-load instructions per wavefront and tile
    constexpr int HALF_TILE = 32 * HD;      // halves of a 32-key K half-tile (8 KB)
    constexpr int TILE = 2 * HALF_TILE;     // 64 keys x 128 dims, K or V^T (16 KB)
    constexpr int VRING = 4 * TILE;         // V ring behind the K ring
    extern __shared__ __attribute__((aligned(16))) half_t smem[];

    const int blk = gridDim.y - 1 - blockIdx.y; // longest rows first
    const int kvh = blockIdx.x;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
    const int head = kvh * G + wave % G;
    const int n = lane % 32, hb = lane / 32;
    const int q0 = blk * 64;          // first row of the workgroup
    const int q0w = q0 + 32 * (wave / G); // first row of this wavefront
    int q_last = q0 + 63;
    if (q_last > T - 1) q_last = T - 1;
    const int nc = (pos0 + q_last) / 32 + 1; // 32-key chunks the workgroup visits
    const int n_tiles = (nc + 1) / 2;
    const int n_plain = (pos0 + q0w + 1) / 32; // chunks that no query of the wavefront has masked keys in

    const int r = q0w + n;
    const int qrow = r < T ? r : T - 1;
    const int qpos = pos0 + r;
    half8_t qf[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[ks] = load8(q + (size_t)qrow * ldq + (size_t)head * HD + 16 * ks + 8 * hb);
    if (ROPE_Q) { // lane (n, hb) holds dims 16 ks + 8 hb .. + 7 of its row: pairs 8 ks + 4 hb .. + 3
        const int rp = qpos < max_pos ? qpos : max_pos - 1;
        const float *cs = table + ((size_t)rp * (HD / 2) + 4 * hb) * 2;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) qf[ks] = rope_rotate8(qf[ks], cs + 16 * ks);
    }

    // tile loads straight into LDS: wave instruction i' = wave + NW t covers 1 KB = 4 K rows or 8 V^T rows; lane l
    // writes 16 bytes at 16 l and fetches the 16-byte chunk of its row that the swizzle puts there
    const __amdgpu_buffer_rsrc_t rs_k = __builtin_amdgcn_make_buffer_rsrc((void *)(kc + (size_t)kvh * max_pos * HD), 0,
                                                                          max_pos * HD * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_v = __builtin_amdgcn_make_buffer_rsrc((void *)(vc + (size_t)kvh * HD * max_pos), 0,
                                                                          HD * max_pos * 2, 0x00020000);
    const int krow_l = 4 * wave + lane / 16;
    const uint32_t kvoff = (uint32_t)krow_l * 256u + (uint32_t)(((lane % 16) ^ (krow_l & 15)) * 16);
    const int vrow_l = 8 * wave + lane / 8;
    const uint32_t vvoff = (uint32_t)vrow_l * (uint32_t)max_pos * 2u + (uint32_t)(((lane % 8) ^ ((vrow_l >> 1) & 7)) * 16);
    auto issue = [&](int tile, int t) __attribute__((always_inline)) { // t < LPT: first half K, second half V
        const int st = tile & 3;
        if (t < LPT / 2) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_k, AP_LDS_PTR(smem + st * TILE + (wave + NW * t) * 512), 16, kvoff,
                                                     (uint32_t)tile * 64u * 256u + (uint32_t)t * (4u * NW * 256u), 0, 0);
        } else {
            const int tt = t - LPT / 2;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_v, AP_LDS_PTR(smem + VRING + st * TILE + (wave + NW * tt) * 512), 16,
                                                     vvoff, (uint32_t)tile * 128u + (uint32_t)tt * (16u * NW) * (uint32_t)max_pos,
                                                     0, 0);
        }
    };
    auto clamp_tile = [&](int tile) __attribute__((always_inline)) { return tile < n_tiles ? tile : n_tiles - 1; };

    // fragment addresses (halves): K rows in the order pi(m) (bits 2 and 3 swapped), 16-byte chunks swizzled
    const int pm = (n & ~0xC) | ((n & 8) >> 1) | ((n & 4) << 1);
    int klane[8], vlane[2][2];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) klane[ks] = pm * 128 + (((2 * ks + hb) ^ (pm & 15)) * 8);
#pragma unroll
    for (int cp = 0; cp < 2; ++cp)
#pragma unroll
        for (int u = 0; u < 2; ++u) vlane[cp][u] = VRING + n * 64 + (((4 * cp + 2 * u + hb) ^ ((n >> 1) & 7)) * 8);

    float16_t S[2];
    ap_u8_t P[2];
    float16_t O[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) O[t][e] = 0.f;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
#pragma unroll
        for (int e = 0; e < 16; ++e) S[b][e] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) P[b][e] = 0u;
    }
    float m_used = -FLT_MAX, l_run = 0.f, sum = 0.f;
    const float c2 = 1.44269504088896341f / sqrtf((float)HD);

    auto xhalf = [&](float x, float &lo, float &hi) __attribute__((always_inline)) {
        auto rr = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
        lo = __uint_as_float(rr[0]);
        hi = __uint_as_float(rr[1]);
    };
    // probabilities of elements 2g, 2g+1 against the reference maximum in use
    auto slice = [&](float16_t &s, ap_u8_t &p, int g) __attribute__((always_inline)) {
        const float nm = -m_used;
        const float p0 = __builtin_amdgcn_exp2f(fmaf(s[2 * g], c2, nm));
        const float p1 = __builtin_amdgcn_exp2f(fmaf(s[2 * g + 1], c2, nm));
        const half2_t h = {(half_t)p0, (half_t)p1};
        p[g] = __builtin_bit_cast(uint32_t, h);
        sum = __builtin_amdgcn_fdot2(h, half2_t{(half_t)1.0f, (half_t)1.0f}, sum, false);
    };
    // The reference maximum only moves when a probability would leave the fp16 range (the row sum turns
    // infinite): then the true running maximum becomes the reference, O^T and the row sum are rescaled and
    // the chunk's probabilities are computed again.  The first chunk always comes through here.
    auto settle = [&](float16_t &s, ap_u8_t &p) __attribute__((always_inline)) {
        const bool bad = !(sum < 3.0e38f);
        if (__builtin_amdgcn_ballot_w64(bad) != 0) {
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); // MFMAs written as text: their result latency is not tracked
            float mx = -FLT_MAX;
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[e]);
            float lo, hi;
            xhalf(mx, lo, hi);
            const float m_new = fmaxf(m_used, fmaxf(lo, hi) * c2);
            const float alpha = __builtin_amdgcn_exp2f(m_used - m_new);
            l_run *= alpha;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) O[t][e] *= alpha;
            m_used = m_new;
            sum = 0.f;
#pragma unroll
            for (int g = 0; g < 8; ++g) slice(s, p, g);
        }
        l_run += sum;
    };
    // causal mask of chunk c on the scores in s: accumulator e is key 32 c + 16 (e / 8) + 8 hb + e % 8
    auto mask = [&](float16_t &s, int c) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int key = 32 * c + 16 * (e / 8) + 8 * hb + (e % 8);
            s[e] = key <= qpos ? s[e] : -FLT_MAX;
        }
    };
    auto pfrag = [&](ap_u8_t &p, int u) __attribute__((always_inline)) {
        ap_u4_t rr = u == 0 ? __builtin_shufflevector(p, p, 0, 1, 2, 3) : __builtin_shufflevector(p, p, 4, 5, 6, 7);
        return __builtin_bit_cast(half8_t, rr);
    };

    // One pipelined iteration on chunk c (PAR = c % 2, PHASE = c % 8): scores of chunk c + 1 into s_nxt, probabilities of chunk c
    // from s_cur into p_cur, O^T += V^T(chunk c - 1) . p_prv.  Every iteration does all three: past the last
    // chunk the scores are computed from a stale ring slot and never used, and in front of the first chunk the
    // probabilities are zero and the V region was cleared.
    // phase_c carries c % 8: the ring slots of the K and V fragments are then compile-time constants and fold into
    // the immediate offsets of the LDS reads (no address arithmetic per read: nine vector-ALU issue slots of about
    // 85 per iteration, which compete with the MFMAs for the issue port).
    auto step = [&](float16_t &s_cur, float16_t &s_nxt, ap_u8_t &p_cur, ap_u8_t &p_prv, int c, auto phase_c,
                    int dma_tile) __attribute__((always_inline)) {
        constexpr int PHASE = decltype(phase_c)::value;
        constexpr int PAR = PHASE & 1;
        constexpr int koff = ((PHASE + 1) & 7) * HALF_TILE;
        constexpr int voff = (((PHASE + 7) & 7) >> 1) * TILE;
        constexpr int RA = 3; // fragments read ahead
        half8_t kf[RA], vf[RA];
        auto rd = [&](int grp) __attribute__((always_inline)) {
            kf[grp % RA] = load8(smem + koff + klane[grp]);
            vf[grp % RA] = load8(smem + voff + vlane[1 - PAR][grp / 4] + (grp % 4) * 2048);
        };
#pragma unroll
        for (int g0 = 0; g0 < RA - 1; ++g0) rd(g0);
        if (c >= n_plain) {
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); // the scores come from MFMAs written as text
            mask(s_cur, c);
        }
        sum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int grp = i / 2;
            if (i % 2 == 0 && grp + RA - 1 < 8) rd(grp + RA - 1);
            if (i % 2 == 0) {
                if (grp == 0) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(s_nxt) : "v"(kf[grp % RA]), "v"(qf[grp]));
                else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(s_nxt) : "v"(kf[grp % RA]), "v"(qf[grp]));
            } else {
                const int t = grp % 4, u = grp / 4;
                asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(O[t]) : "v"(vf[grp % RA]), "v"(pfrag(p_prv, u)));
            }
            if (i % 2 == 1) slice(s_cur, p_cur, grp);
            if (i % 8 == 3) issue(dma_tile, (1 - PAR) * (LPT / 2) + i / 8);
            __builtin_amdgcn_sched_barrier(0);
        }
        settle(s_cur, p_cur);
    };
    // tile (c + 1) / 2 must have landed before the scores of chunk c + 1 (c odd): at most the loads of the tile
    // after it stay in flight; behind the barrier the stage of tile (c + 1) / 2 - 2 is free
    auto tile_barrier = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(LPT) : "memory"); };

    // tiles 0 and 1 and the K half of tile 2 (chunk 0 issues its V half); the V region that the second product
    // of the first iteration reads (tile 3, with zero probabilities) must not hold NaN or infinity patterns
    {
        const half8_t z8 = {(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
#pragma unroll
        for (int i = 0; i < TILE / 8 / THREADS; ++i) store8(smem + VRING + 3 * TILE + (tid + THREADS * i) * 8, z8);
    }
#pragma unroll
    for (int t = 0; t < LPT; ++t) issue(0, t);
#pragma unroll
    for (int t = 0; t < LPT; ++t) issue(clamp_tile(1), t);
#pragma unroll
    for (int t = 0; t < LPT / 2; ++t) issue(clamp_tile(2), t);
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(LPT + LPT / 2) : "memory");

    // scores of chunk 0
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
        const half8_t kf = load8(smem + klane[ks]);
        if (ks == 0) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(S[0]) : "v"(kf), "v"(qf[ks]));
        else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(S[0]) : "v"(kf), "v"(qf[ks]));
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // Iterations come in pairs, so that the two score and probability sets keep their roles.  With an odd number
    // of chunks the last iteration works on chunk nc, whose keys lie behind every query of the block: masked,
    // its probabilities are zero, and the second product of the last real chunk rides on it.
    // Eight iterations per trip (the period of the K ring), left after any pair.
    int dma_tile = clamp_tile(2);
    for (int c = 0; c < nc; c += 8) {
#define AP_PAIR(PH)                                                                               \
        step(S[0], S[1], P[0], P[1], c + PH, std::integral_constant<int, PH>{}, dma_tile);          \
        tile_barrier();                                                                            \
        dma_tile = clamp_tile((c + PH) / 2 + 3);                                                   \
        step(S[1], S[0], P[1], P[0], c + PH + 1, std::integral_constant<int, PH + 1>{}, dma_tile);
        AP_PAIR(0)
        if (c + 2 >= nc) break;
        AP_PAIR(2)
        if (c + 4 >= nc) break;
        AP_PAIR(4)
        if (c + 6 >= nc) break;
        AP_PAIR(6)
#undef AP_PAIR
    }
    if (!(nc & 1)) { // second product of the last chunk
        const int voff = (((nc - 1) >> 1) & 3) * TILE;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const half8_t vf = load8(smem + voff + vlane[1][u] + t * 2048);
                asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(O[t]) : "v"(vf), "v"(pfrag(P[1], u)));
            }
    }
    asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");

    // O^T lane l: query q0w + l%32, dims 32 t + 8 (e/4) + 4 (l/32) + e%4
    {
        float lo, hi;
        xhalf(l_run, lo, hi);
        if (r < T) {
            const float inv = 1.0f / (lo + hi);
            half_t *orow = out + (size_t)r * ldo + (size_t)head * HD;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    half4_t v;
#pragma unroll
                    for (int i = 0; i < 4; ++i) v[i] = (half_t)(O[t][4 * e4 + i] * inv);
                    *reinterpret_cast<half4_t *>(orow + 32 * t + 8 * e4 + 4 * hb) = v;
                }
        }
    }
}

template <bool ROPE_Q>
static int launch_prefill_pipe(const half_t *q, int ldq, const half_t *kc, const half_t *vc, half_t *out, int ldo, int T,
                               int pos0, int n_kv_heads, int max_pos, const float *table, hipStream_t s) {
    dim3 grid(n_kv_heads, (T + 63) / 64);
    const size_t smem = 8 * 64 * 128 * sizeof(half_t); // four stages of a K and a V^T tile
    auto kern = attn_prefill_pipe_kernel<4, ROPE_Q>;
    static std::atomic<uint64_t> attr_done{0};
    int rc = llm_ensure_max_smem((const void *)kern, smem, attr_done);
    if (rc != LLM_OK) return rc;
    kern<<<grid, dim3(512), smem, s>>>(q, ldq, kc, vc, out, ldo, T, pos0, max_pos, table);
    LLM_LAUNCH_CHECK("attn_prefill_pipe_kernel");
    return LLM_OK;
}

template <int HD, int G>
static int launch_prefill(const half_t *q, int ldq, const half_t *kc, const half_t *vc, half_t *out, int ldo,
                          int T, int pos0, int n_kv_heads, int max_pos, hipStream_t s) {
    constexpr int AP_QT = G >= 8 ? 1 : 2; // 32-row query tiles per workgroup (at most 8 wavefronts)
    const int n_qt = (T + AP_BQ - 1) / AP_BQ;
    dim3 grid(n_kv_heads, (n_qt + AP_QT - 1) / AP_QT);
    const size_t smem = sizeof(half_t) * 2 * ((size_t)AP_BKEY * (HD + 8) + (size_t)HD * (AP_BKEY + 8));
    auto kern = attn_prefill_kernel<HD, G, AP_QT>;
    static std::atomic<uint64_t> attr_done{0};
    if (smem > 48 * 1024) {
        int rc = llm_ensure_max_smem((const void *)kern, smem, attr_done);
        if (rc != LLM_OK) return rc;
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
    // the pipelined kernel addresses one KV head's cache through a 32-bit buffer descriptor
    if (head_dim == 128 && G == 4 && T >= AP_PIPE_MIN_ROWS && (size_t)max_pos * 128 * sizeof(half_t) < (1ull << 31))
        return launch_prefill_pipe<false>(qp, ldq, kp, vp, op, ldo, T, pos0, n_kv_heads, max_pos, nullptr, s);
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

// The shapes the pipelined kernel serves: the only ones for which the attention rotates the queries itself.
static bool prefill_pipe_shape(int T, int n_heads, int n_kv_heads, int head_dim, int max_pos) {
    return n_kv_heads > 0 && n_heads == 4 * n_kv_heads && head_dim == 128 && T >= AP_PIPE_MIN_ROWS &&
           (size_t)max_pos * 128 * sizeof(half_t) < (1ull << 31);
}

extern "C" int llm_attn_prefill_rope_q_supported(int T, int n_heads, int n_kv_heads, int head_dim, int max_pos) {
    return prefill_pipe_shape(T, n_heads, n_kv_heads, head_dim, max_pos) ? 1 : 0;
}

extern "C" int llm_attn_prefill_rope_q(const uint16_t *q, int ldq, const uint16_t *kc, const uint16_t *vc, uint16_t *out, int ldo,
                                       int T, int pos0, const float *table, int n_heads, int n_kv_heads, int head_dim,
                                       int max_pos, llm_stream_t stream) {
    LLM_REQUIRE(q && kc && vc && out && table, "llm_attn_prefill_rope_q: null pointer");
    LLM_REQUIRE(prefill_pipe_shape(T, n_heads, n_kv_heads, head_dim, max_pos),
                "llm_attn_prefill_rope_q: %d rows, heads %d/%d of %d are not covered (llm_attn_prefill_rope_q_supported)", T, n_heads,
                n_kv_heads, head_dim);
    LLM_REQUIRE(pos0 >= 0 && pos0 + T <= max_pos, "llm_attn_prefill_rope_q: rows %d..%d of %d", pos0, pos0 + T, max_pos);
    LLM_REQUIRE(max_pos % 64 == 0, "llm_attn_prefill_rope_q: max_pos=%d must be a multiple of 64", max_pos);
    LLM_REQUIRE(ldq % 8 == 0 && ldq >= n_heads * head_dim && ldo % 4 == 0 && ldo >= n_heads * head_dim,
                "llm_attn_prefill_rope_q: ldq=%d ldo=%d", ldq, ldo);
    LLM_REQUIRE(aligned16(q) && aligned16(kc) && aligned16(vc) && aligned16(table) && ((uintptr_t)out & 7u) == 0,
                "llm_attn_prefill_rope_q: pointers must be 16-byte aligned");
    return launch_prefill_pipe<true>((const half_t *)q, ldq, (const half_t *)kc, (const half_t *)vc, (half_t *)out, ldo, T, pos0,
                                     n_kv_heads, max_pos, table, (hipStream_t)stream);
}
