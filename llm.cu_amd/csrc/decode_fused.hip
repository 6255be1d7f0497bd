// One decode token of the whole model in one launch (positions below 512).
//
// A decode step is a chain of bandwidth-bound one-row projections (QKV, O, gate/up, down per layer, then
// the LM head) with a small attention between QKV and O.  As separate launches every link of the chain
// costs a launch, a first trip to HBM and a drained pipeline: HBM idles for 2-3 us between any two
// kernels and for the whole attention.  Here one resident workgroup per CU walks through all phases:
//
//   workgroups 0 .. n_attn-1            the attention of every layer (attn_decode_body, one KV head and one
//                                       quarter of the head dims each, as in the stand-alone kernel)
//   workgroups n_attn .. grid-1         the projections: phase p = 4*layer + {0 QKV, 1 O, 2 gate/up, 3 down},
//                                       then the LM head
//
// A projection wavefront owns groups of four adjacent weight rows (group g = slot + n_slots * i) and
// streams them through a ring of three register stages (four 16-byte loads per lane and stage: a 2048-k
// span of a row, the lane mapping and the accumulation order of the stand-alone GEMV, so the sums are the
// same bits).  The ring runs ahead across phase boundaries: while a workgroup waits for the input vector of
// the next phase, the first spans of that phase's weights are already on their way.
//
// Hand-over between phases without counters, fences or grid barriers: every vector that one phase
// produces and the next consumes (qkv, attention output, x after O, the FFN hidden vector, x after down)
// has its own buffer per layer, armed with a 16-bit pattern that no phase writes as a value (DF_EMPTY, a
// NaN; a result with those bits is stored with the lowest bit cleared).  Producers store four results at a
// time as one 8-byte device-scope (write-through) store; consumers read the vector with device-scope loads
// until no word holds the pattern.  The data is its own flag.  Two sets of buffers alternate from token to
// token: a launch uses `ring_cur` and re-arms `ring_next`, which the previous launch used.
//
// Every workgroup is resident from the start (grid <= number of CUs, one workgroup per CU) and all waits
// are on data whose producers are running, so the chain cannot deadlock; each wait is bounded anyway
// (DF_POLL_LIMIT rounds, then the workgroup carries on and counts a timeout for the host to see).
//
// Arithmetic is that of the separate kernels (rms_device.hpp for the norms, the GEMV's dot order,
// attn_decode_body for the attention): the logits equal the per-kernel path bit for bit.
#include <cmath>
#include <type_traits>

#include "common.hpp"

#include "attn_decode_body.hpp"
#include "rms_device.hpp"

#define DF_THREADS AD_THREADS
#define DF_WAVES AD_WAVES
#define DF_U 4              // 16-byte loads per lane and stage
#define DF_SPAN (512 * DF_U)
#define DF_STAGES 3
#define DF_EMPTY 0xFFFFu
#define DF_POLL_LIMIT (1 << 18)
#define DF_XS_HALVES 16384  // LDS staging of a phase's input vector (the FFN width is the widest)
#define DF_CTRL_WAVES 4     // wavefronts per projection workgroup that poll, stage and store
#define DF_BLOCK (DF_THREADS + DF_CTRL_WAVES * WAVE)
#define DF_NORM_R 16        // RMSNorm by one wavefront: d / 4 / 64 slots per lane (d <= 4096)
#define DF_RES_PRE 2        // residual words a control wavefront prefetches per phase
#define DF_COPY_R 8         // 8-byte words per lane and round when a vector is copied to LDS
#define DF_MAX_ROUNDS 96    // rows per streaming wavefront and phase, at most (the LM head has the most)

enum { PH_QKV = 0, PH_O = 1, PH_GU = 2, PH_DOWN = 3, PH_LM = 4 };

struct DfLayer { // llm_decode_layer of the C-ABI
    const half_t *in_ln, *wqkv, *wo, *post_ln, *wg, *wu, *wd;
    half_t *kc, *vc;
};

struct DfArgs {
    const DfLayer *layers;
    int L, d, qd, qkv, F, vocab;
    int n_heads, n_kv_heads, head_dim, max_pos;
    double eps;
    const float *rope_table;
    const int32_t *pos_dev, *tokens_dev;
    const half_t *embed, *final_gain, *lm_head;
    half_t *logits;
    unsigned long long *cand;
    uint16_t *ring_cur, *ring_next;
    int *timeouts;
    int n_attn, p_begin, p_end;
};

// per layer in a ring set (halves): qkv | attn | x1 (after O) | h | x2 (after down)
__device__ __forceinline__ size_t df_per_layer(const DfArgs &a) { return (size_t)a.qkv + a.qd + 2 * (size_t)a.d + a.F; }
__device__ __forceinline__ uint16_t *df_vec(const DfArgs &a, int l, int which) {
    uint16_t *b = a.ring_cur + df_per_layer(a) * l;
    return which == 0 ? b : which == 1 ? b + a.qkv : which == 2 ? b + a.qkv + a.qd : which == 3 ? b + a.qkv + a.qd + a.d
                                                                                              : b + a.qkv + a.qd + a.d + a.F;
}

struct DfPhase {
    const half_t *w, *w2;   // weights [N, K] (w2: the up matrix of gate/up)
    const uint16_t *in;     // input vector (hand-over buffer or the embedding row), K halves
    const half_t *gain;     // RMSNorm gains applied while staging `in`, or null
    const uint16_t *res;    // residual vector (N halves) or null
    uint16_t *out;          // output vector (hand-over buffer; PH_LM: the logits)
    int K, N, type;
};

__device__ __forceinline__ DfPhase df_phase(const DfArgs &a, int p, const uint16_t *x0) {
    DfPhase ph;
    ph.w2 = nullptr;
    ph.gain = nullptr;
    ph.res = nullptr;
    if (p >= 4 * a.L) {
        ph.type = PH_LM;
        ph.w = a.lm_head;
        ph.in = df_vec(a, a.L - 1, 4);
        ph.gain = a.final_gain;
        ph.out = reinterpret_cast<uint16_t *>(a.logits);
        ph.K = a.d;
        ph.N = a.vocab;
        return ph;
    }
    const int l = p >> 2;
    const DfLayer &ly = a.layers[l];
    const uint16_t *xin = l == 0 ? x0 : df_vec(a, l - 1, 4); // the residual stream entering the layer
    ph.type = p & 3;
    switch (p & 3) {
    case PH_QKV:
        ph.w = ly.wqkv, ph.in = xin, ph.gain = ly.in_ln, ph.out = df_vec(a, l, 0), ph.K = a.d, ph.N = a.qkv;
        break;
    case PH_O:
        ph.w = ly.wo, ph.in = df_vec(a, l, 1), ph.res = xin, ph.out = df_vec(a, l, 2), ph.K = a.qd, ph.N = a.d;
        break;
    case PH_GU:
        ph.w = ly.wg, ph.w2 = ly.wu, ph.in = df_vec(a, l, 2), ph.gain = ly.post_ln, ph.out = df_vec(a, l, 3), ph.K = a.d,
        ph.N = a.F;
        break;
    default:
        ph.w = ly.wd, ph.in = df_vec(a, l, 3), ph.res = df_vec(a, l, 2), ph.out = df_vec(a, l, 4), ph.K = a.F, ph.N = a.d;
        break;
    }
    return ph;
}

__device__ __forceinline__ bool df_has_empty(unsigned long long v) {
    return (v & 0xFFFFull) == DF_EMPTY || ((v >> 16) & 0xFFFFull) == DF_EMPTY || ((v >> 32) & 0xFFFFull) == DF_EMPTY ||
           (v >> 48) == DF_EMPTY;
}

// steps of a phase, the same for every wavefront: rounds x steps per row, rounded up to whole ring turns
// so that the stage a step uses is a compile-time constant on both the issuing and the consuming side
struct DfWork {
    int spr, nsteps, padded; // steps per row, steps, steps incl. padding
};
__device__ __forceinline__ DfWork df_work(const DfPhase &ph, int wtotal) {
    DfWork w;
    const int spans = (ph.K + DF_SPAN - 1) / DF_SPAN;
    w.spr = ph.w2 ? spans : (spans + 1) / 2;
    const int rounds = (ph.N + wtotal - 1) / wtotal;
    w.nsteps = rounds * w.spr;
    w.padded = (w.nsteps + DF_STAGES - 1) / DF_STAGES * DF_STAGES;
    return w;
}

// One 16-byte weight load as an instruction (streamed once: nt), so that the compiler neither counts it nor
// waits for it: df_wait_stage does, with the count the loop's structure fixes.
template <int OFF> __device__ __forceinline__ void df_load(half8_t &dst, const half_t *p) {
    asm volatile("global_load_dwordx4 %0, %1, off offset:%2 nt" : "=v"(dst) : "v"(p), "n"(OFF));
}
// The eight loads of one ring stage have completed when at most the 16 loads of the two younger stages are
// still outstanding (vector memory loads return in order).  The registers are operands so that no use of
// them can move above the wait.
__device__ __forceinline__ void df_wait_stage(half8_t (&b)[2][DF_U]) {
    asm volatile("s_waitcnt vmcnt(16)"
                 : "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[0][2]), "+v"(b[0][3]), "+v"(b[1][0]), "+v"(b[1][1]), "+v"(b[1][2]),
                   "+v"(b[1][3]));
}

// LDS-only ordering between the wavefronts of a workgroup (no wait on global memory: the weight loads in
// flight must stay in flight)
__device__ __forceinline__ void df_lds_release() { __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local"); }
__device__ __forceinline__ void df_lds_acquire() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local"); }
__device__ __forceinline__ int df_lds_load(const int *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void df_lds_store(int *p, int v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

template <int HD, int G, int DSN>
__global__ __launch_bounds__(DF_BLOCK) void decode_fused_kernel(const DfArgs a) {
    // projections: the staged input vector of phase p lives in xsb[p & 1] (a phase's vector may be staged, piece
    // by piece, while the previous phase is still reading its own)
    __shared__ __attribute__((aligned(16))) half_t xsb[2][DF_XS_HALVES];
    half_t *const xs = xsb[0]; // the attention workgroups carve their scratch out of the first one
    __shared__ float red[DF_THREADS + 1];
    __shared__ unsigned long long best[DF_WAVES];
    // finished rows, [round][streaming wavefront]: (sequence number << 16) | fp16 bits in one word, so that a
    // reader that sees the sequence number it waits for has the value too (no second location to order)
    __shared__ int rowslot[DF_MAX_ROUNDS][DF_WAVES];
    __shared__ int staged;   // control wavefronts that have staged, cumulative over phases
    __shared__ int rawready; // phase (+1) whose raw input vector the first control wavefront has put into LDS
    const int wg = blockIdx.x, tid = threadIdx.x;
    const int wave = tid / WAVE, lane = tid % WAVE;
    int pos = *a.pos_dev;
    pos = pos < 0 ? 0 : pos;
    pos = pos > a.max_pos - 1 ? a.max_pos - 1 : pos;
    pos = pos > AD_LS - 1 ? AD_LS - 1 : pos; // one attention span; the host uses this kernel below AD_LS only

    // re-arm the other set of hand-over buffers (the previous launch used it; nobody reads it now)
    {
        const size_t n16 = df_per_layer(a) * a.L / 8; // 16-byte units
        uint4_t *nx = reinterpret_cast<uint4_t *>(a.ring_next);
        const uint32_t e2 = DF_EMPTY | (DF_EMPTY << 16);
        for (size_t i = (size_t)wg * DF_BLOCK + tid; i < n16; i += (size_t)gridDim.x * DF_BLOCK) nx[i] = uint4_t{e2, e2, e2, e2};
    }

    if (wg < a.n_attn) {
        // ---- attention of every layer in the phase range (eight wavefronts; the others have nothing to do) ----
        if (wave >= DF_WAVES) return;
        float *sc = reinterpret_cast<float *>(xs);                       // G * AD_LS floats
        half_t *qs = xs + 2 * G * AD_LS;                                 // G * HD
        half_t *knew = qs + G * HD, *vnew = knew + HD, *qkv_l = vnew + HD; // HD, HD, (G + 2) * HD
        static_assert(2 * G * AD_LS + G * HD + 2 * HD + (G + 2) * HD <= DF_XS_HALVES, "attention LDS");
        float *s_m = red, *s_l = red + G;
        int *s_last = reinterpret_cast<int *>(red + 2 * G);
        const int kvh = wg % a.n_kv_heads, y = wg / a.n_kv_heads;
        for (int l = 0; l < a.L; ++l) {
            if (4 * l + PH_O < a.p_begin || 4 * l + PH_O >= a.p_end) continue;
            AdArgs ad = {};
            ad.q = reinterpret_cast<const half_t *>(df_vec(a, l, 0));
            ad.kc = a.layers[l].kc;
            ad.vc = a.layers[l].vc;
            ad.out = reinterpret_cast<half_t *>(df_vec(a, l, 1));
            ad.table = a.rope_table;
            ad.n_kv_heads = a.n_kv_heads;
            ad.max_pos = a.max_pos;
            ad.splits = 1;
            __syncthreads(); // LDS of the previous layer is free
            attn_decode_body<HD, G, true, HD / DSN, AD_LS, false, true, true>(ad, sc, qs, knew, vnew, s_m, s_l, s_last, pos, 1, 0,
                                                                              y * (HD / DSN), y == 0, kvh, qkv_l, a.timeouts);
        }
        return;
    }

    // ---- projections ---------------------------------------------------------------------------
    // Eight streaming wavefronts pull weight rows and reduce them against the staged input vector; their loop
    // holds no global memory operation other than the weight loads, so those stay in flight across rows and
    // phases.  The control wavefronts do everything that has to wait for other workgroups: they read the
    // phase's input vector until it is complete and stage it in LDS (normalised where the phase starts with an
    // RMSNorm), and they collect the finished rows from LDS, add the residual and store them for the next
    // phase.  The two sides talk through LDS only (progress counters, no workgroup barrier).
    const int wgp = wg - a.n_attn;
    const int wtotal = ((int)gridDim.x - a.n_attn) * DF_WAVES; // rows per round over all workgroups
    int tok = a.tokens_dev[pos];
    tok = tok < 0 ? 0 : (tok >= a.vocab ? a.vocab - 1 : tok); // the host validates ids; this keeps the read in bounds
    const uint16_t *x0 = reinterpret_cast<const uint16_t *>(a.embed) + (size_t)tok * a.d;
    for (int i = tid; i < DF_MAX_ROUNDS * DF_WAVES; i += DF_BLOCK) (&rowslot[0][0])[i] = 0;
    if (tid == 0) staged = 0, rawready = 0;
    __syncthreads(); // the only workgroup barrier of the projection part

    if (wave < DF_WAVES) {
        // ===== streaming wavefront ==============================================================
        // Round i of a phase: wavefront v of projection workgroup b owns row (i*nproj + b)*8 + v.  A step moves
        // two 2048-k spans of that row (gate/up: one span of each matrix): always eight 16-byte loads per lane,
        // also for padding steps, rows past the end and spans past K (those re-read the start of the matrix;
        // the staged vector is zero there), so the number of loads in flight is the same at every point of the
        // loop.  The loads are written as instructions and waited for with an explicit count: three stages
        // ring, 16 younger loads may still be in flight when a stage is consumed.  Nothing else in this loop
        // touches global memory.
        half8_t buf[DF_STAGES][2][DF_U];
        int ip = a.p_begin, istep = 0;
        DfPhase iph = df_phase(a, ip, x0);
        DfWork iw = df_work(iph, wtotal);
        auto issue = [&](auto STAGE) {
            constexpr int S = decltype(STAGE)::value;
            while (ip < a.p_end - 1 && istep >= iw.padded) {
                ++ip;
                istep = 0;
                iph = df_phase(a, ip, x0);
                iw = df_work(iph, wtotal);
            }
            const int round = istep / iw.spr, st = istep - round * iw.spr;
            const size_t row = (size_t)wgp * DF_WAVES + wave + (size_t)round * wtotal;
            const bool live = istep < iw.nsteps && row < (size_t)iph.N;
            const int sp0 = iph.w2 ? st : 2 * st, sp1 = iph.w2 ? st : 2 * st + 1;
            const half_t *w1 = iph.w2 ? iph.w2 : iph.w;
            const half_t *b0 = iph.w + (live ? row * iph.K : 0), *b1 = w1 + (live ? row * iph.K : 0);
            const int k0 = sp0 * DF_SPAN + lane * 8, k1 = sp1 * DF_SPAN + lane * 8;
            // one instruction sequence for every case: a load past the end of the row (ragged K, the odd span
            // of a row with an odd number of spans, padding steps) reads the row's start instead
            df_load<0>(buf[S][0][0], b0 + (live && k0 < iph.K ? k0 : 0));
            df_load<0>(buf[S][0][1], b0 + (live && k0 + 512 < iph.K ? k0 + 512 : 0));
            df_load<0>(buf[S][0][2], b0 + (live && k0 + 1024 < iph.K ? k0 + 1024 : 0));
            df_load<0>(buf[S][0][3], b0 + (live && k0 + 1536 < iph.K ? k0 + 1536 : 0));
            df_load<0>(buf[S][1][0], b1 + (live && k1 < iph.K ? k1 : 0));
            df_load<0>(buf[S][1][1], b1 + (live && k1 + 512 < iph.K ? k1 + 512 : 0));
            df_load<0>(buf[S][1][2], b1 + (live && k1 + 1024 < iph.K ? k1 + 1024 : 0));
            df_load<0>(buf[S][1][3], b1 + (live && k1 + 1536 < iph.K ? k1 + 1536 : 0));
            ++istep;
        };
        // One flat loop over the steps of all phases; the consuming side runs one ring turn (three steps)
        // behind the issuing side.  There is no separate pipeline prologue: a register that a load in flight
        // will write must never be copied, and values that enter a loop from outside are what compilers copy.
        int cp = a.p_begin, cstep = 0, cum = 0; // consume cursor: phase, step of its padded steps; rounds before it
        DfPhase ph = df_phase(a, cp, x0);
        DfWork w = df_work(ph, wtotal);
        float acc0 = 0.f, acc1 = 0.f;
        unsigned long long mine = 0ull;
        int round = 0, st = 0;
        auto consume = [&](auto STAGE) {
            constexpr int S = decltype(STAGE)::value;
            df_wait_stage(buf[S]); // this stage's eight loads have landed (16 younger ones may be in flight)
            if (cp >= a.p_end) return;
            if (cstep == 0) {
                // phase entry: its input vector is in LDS once every control wavefront has done its share
                const int want = DF_CTRL_WAVES * (cp - a.p_begin + 1);
                while (df_lds_load(&staged) < want) __builtin_amdgcn_s_sleep(1);
                df_lds_acquire();
            }
            if (cstep < w.nsteps) {
                const int sp0 = ph.w2 ? st : 2 * st, sp1 = ph.w2 ? st : 2 * st + 1;
                const half_t *xv = xsb[cp & 1];
                const half_t *x0p = xv + sp0 * DF_SPAN + lane * 8, *x1p = xv + sp1 * DF_SPAN + lane * 8;
#pragma unroll
                for (int u = 0; u < DF_U; ++u) acc0 = dot8(buf[S][0][u], load8(x0p + u * 512), acc0);
                if (ph.w2) {
#pragma unroll
                    for (int u = 0; u < DF_U; ++u) acc1 = dot8(buf[S][1][u], load8(x1p + u * 512), acc1);
                } else {
#pragma unroll
                    for (int u = 0; u < DF_U; ++u) acc0 = dot8(buf[S][1][u], load8(x1p + u * 512), acc0);
                }
                if (++st == w.spr) {
                    st = 0;
                    // the row is complete: hand it to the control wavefronts through LDS
                    const size_t row = (size_t)wgp * DF_WAVES + wave + (size_t)round * wtotal;
                    const float s0 = wave_sum(acc0);
                    const float s1 = ph.w2 ? wave_sum(acc1) : 0.f;
                    acc0 = acc1 = 0.f;
                    const half_t val = ph.type == PH_GU ? swiglu_to_half(s0, s1) : (half_t)s0;
                    if (ph.type == PH_LM && row < (size_t)ph.N) {
                        const unsigned long long c = pack_candidate(val, (int)row);
                        mine = c > mine ? c : mine;
                    }
                    ++round;
                    if (lane == 0) {
                        if (ph.type == PH_LM) {
                            best[wave] = mine;
                            df_lds_release();
                        }
                        df_lds_store(&rowslot[round - 1][wave], ((cum + round) << 16) | __builtin_bit_cast(uint16_t, val));
                    }
                }
            }
            if (++cstep == w.padded) { // next phase
                cum += round;
                round = 0;
                cstep = 0;
                ++cp;
                if (cp < a.p_end) {
                    ph = df_phase(a, cp, x0);
                    w = df_work(ph, wtotal);
                }
            }
        };
        for (int turn = 0; cp < a.p_end; ++turn) {
            if (turn) consume(std::integral_constant<int, 0>{});
            issue(std::integral_constant<int, 0>{});
            if (turn) consume(std::integral_constant<int, 1>{});
            issue(std::integral_constant<int, 1>{});
            if (turn) consume(std::integral_constant<int, 2>{});
            issue(std::integral_constant<int, 2>{});
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the loads issued past the last step
        return;
    }

    // ===== control wavefronts ======================================================================
    const int cw = wave - DF_WAVES; // 0 .. DF_CTRL_WAVES-1
    int cum = 0;
    for (int p = a.p_begin; p < a.p_end; ++p) {
        const DfPhase ph = df_phase(a, p, x0);
        const DfWork w = df_work(ph, wtotal);
        const int rounds = w.nsteps / w.spr;
        half_t *const xsp = xsb[p & 1];
        // ---- stage the input vector: wait until its producers have written all of it -------------------
        // (into the buffer that the phase before the previous one used: every streaming wavefront is past that
        // phase, because this wavefront has already stored rows of the previous phase)
        {
            const unsigned long long *src = reinterpret_cast<const unsigned long long *>(ph.in);
            const int n8 = ph.K / 4; // 8-byte words = RMSNorm slots
            if (ph.gain) {
                // RMSNorm in the reference's order (slot j of lane t = elements 4 * (t + 64 * j)).  Every control
                // wavefront reads the whole vector and takes the sum of squares for itself (same tree, same bits);
                // each then normalises a quarter of the slots.  The gains are asked for before the wait.
                RmsRow<DF_NORM_R> r;
                const int R = n8 >= WAVE ? n8 / WAVE : 1;
                r.R = lane < n8 ? R : 0;
#pragma unroll
                for (int j = 0; j < DF_NORM_R; ++j)
                    if (j < r.R && j % DF_CTRL_WAVES == cw)
                        r.g[j] = *reinterpret_cast<const half4_t *>(ph.gain + 4 * (size_t)(lane + WAVE * j));
                // One control wavefront per workgroup reads the vector from memory (hundreds of wavefronts polling
                // the same 8 KB crowd the few channels that hold it) and passes the raw words on through LDS,
                // behind the normalised vector (K <= 4096 halves there, the raw copy sits at 8192).
                unsigned long long *raw = reinterpret_cast<unsigned long long *>(xsp + DF_XS_HALVES / 2);
                if (cw == 0) {
                    int spins = 0;
                    for (;;) {
                        bool empty = false;
#pragma unroll
                        for (int j = 0; j < DF_NORM_R; ++j) {
                            if (j < r.R) {
                                const unsigned long long v =
                                    __hip_atomic_load(src + lane + WAVE * j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                empty |= df_has_empty(v);
                                r.x[j] = __builtin_bit_cast(half4_t, v);
                            }
                        }
                        if (!__any(empty)) break;
                        if (++spins > DF_POLL_LIMIT) {
                            if (lane == 0) atomicAdd(a.timeouts, 1);
                            break;
                        }
                        __builtin_amdgcn_s_sleep(2);
                    }
#pragma unroll
                    for (int j = 0; j < DF_NORM_R; ++j)
                        if (j < r.R) raw[lane + WAVE * j] = __builtin_bit_cast(unsigned long long, r.x[j]);
                    df_lds_release();
                    if (lane == 0) df_lds_store(&rawready, p + 1);
                } else {
                    while (df_lds_load(&rawready) != p + 1) __builtin_amdgcn_s_sleep(1);
                    df_lds_acquire();
#pragma unroll
                    for (int j = 0; j < DF_NORM_R; ++j)
                        if (j < r.R) r.x[j] = __builtin_bit_cast(half4_t, raw[lane + WAVE * j]);
                }
                const float ss = rms_sum_squares<WAVE, DF_NORM_R>(r, ph.K, red, lane);
                const float rms = rms_from_ss(ss, ph.K, a.eps);
#pragma unroll
                for (int j = 0; j < DF_NORM_R; ++j) {
                    if (j < r.R && j % DF_CTRL_WAVES == cw) {
                        half4_t o;
#pragma unroll
                        for (int k = 0; k < 4; ++k) o[k] = (half_t)(((float)r.x[j][k] * (float)r.g[j][k]) / rms);
                        *reinterpret_cast<half4_t *>(xsp + 4 * (size_t)(lane + WAVE * j)) = o;
                    }
                }
            } else {
                // plain copy, the control wavefronts share the words
                for (int c0 = cw * WAVE; c0 < n8; c0 += DF_CTRL_WAVES * WAVE * DF_COPY_R) {
                    unsigned long long v[DF_COPY_R];
                    int spins = 0;
                    for (;;) {
                        bool empty = false;
#pragma unroll
                        for (int j = 0; j < DF_COPY_R; ++j) {
                            const int c = c0 + lane + DF_CTRL_WAVES * WAVE * j;
                            v[j] = c < n8 ? __hip_atomic_load(src + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
                        }
#pragma unroll
                        for (int j = 0; j < DF_COPY_R; ++j) empty |= df_has_empty(v[j]);
                        if (!__any(empty)) break;
                        if (++spins > DF_POLL_LIMIT) {
                            if (lane == 0) atomicAdd(a.timeouts, 1);
                            break;
                        }
                        __builtin_amdgcn_s_sleep(1);
                    }
#pragma unroll
                    for (int j = 0; j < DF_COPY_R; ++j) {
                        const int c = c0 + lane + DF_CTRL_WAVES * WAVE * j;
                        if (c < n8) reinterpret_cast<unsigned long long *>(xsp)[c] = v[j];
                    }
                }
            }
            // zeros behind the vector up to the end of the last step (the streaming loop multiplies whole steps)
            {
                const int end = w.spr * (ph.w2 ? 1 : 2) * DF_SPAN;
                for (int c = ph.K + (cw * WAVE + lane) * 8; c < end; c += DF_CTRL_WAVES * WAVE * 8)
                    store8(xsp + c, half8_t{0, 0, 0, 0, 0, 0, 0, 0});
            }
            df_lds_release();
            if (lane == 0) __hip_atomic_fetch_add(&staged, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        // ---- collect the rows of the phase as the streaming wavefronts finish them ---------------------
        // round i, half h (rows +4h .. +4h+3 of the workgroup's eight) is handled by control wavefront
        // (2i + h) % DF_CTRL_WAVES, lane 0
        // the residuals of this wavefront's first items are asked for up front (one trip to memory for all of
        // them instead of one per item)
        unsigned long long respre[DF_RES_PRE];
#pragma unroll
        for (int q = 0; q < DF_RES_PRE; ++q) {
            const int item = cw + DF_CTRL_WAVES * q;
            const size_t row0 = (size_t)wgp * DF_WAVES + (size_t)(item >> 1) * wtotal + 4 * (item & 1);
            respre[q] = 0ull;
            if (ph.res && lane == 0 && item < 2 * rounds && row0 < (size_t)ph.N)
                respre[q] = __hip_atomic_load(reinterpret_cast<const unsigned long long *>(ph.res + row0), __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
        }
        for (int item = cw, q = 0; item < 2 * rounds; item += DF_CTRL_WAVES, ++q) {
            const int round = item >> 1, half = item & 1;
            const size_t row0 = (size_t)wgp * DF_WAVES + (size_t)round * wtotal + 4 * half;
            if (row0 >= (size_t)ph.N) continue; // rows past the end (last round only)
            unsigned long long resq = q == 0 ? respre[0] : q == 1 ? respre[1] : 0ull;
            if (ph.res && lane == 0 && q >= DF_RES_PRE)
                resq = __hip_atomic_load(reinterpret_cast<const unsigned long long *>(ph.res + row0), __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
            int spins = 0, slot[4];
            for (;;) {
                bool ready = true;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    slot[i] = df_lds_load(&rowslot[round][4 * half + i]);
                    ready &= (slot[i] >> 16) == cum + round + 1;
                }
                if (ready) break;
                if (++spins > DF_POLL_LIMIT * 16) {
                    if (lane == 0) atomicAdd(a.timeouts, 1);
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
            if (lane == 0) {
                unsigned long long packed = 0ull;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    half_t h = __builtin_bit_cast(half_t, (uint16_t)(slot[i] & 0xFFFF));
                    if (ph.res) { // fp16(fp16(sum) + residual): the reference's add_norm on the stored projection
                        const half_t rv = __builtin_bit_cast(half_t, (uint16_t)(resq >> (16 * i)));
                        h = (half_t)((float)h + (float)rv);
                    }
                    uint16_t bits = __builtin_bit_cast(uint16_t, h);
                    if (ph.type != PH_LM && bits == DF_EMPTY) bits = DF_EMPTY - 1; // reserved for "not written yet"
                    packed |= (unsigned long long)bits << (16 * i);
                }
                unsigned long long *dst = reinterpret_cast<unsigned long long *>(ph.out + row0);
                if (ph.type == PH_LM) *dst = packed;
                else __hip_atomic_store(dst, packed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        cum += rounds;
        if (ph.type == PH_LM && cw == 0) { // one argmax candidate per workgroup, once every wavefront is through
            int spins = 0;
            for (;;) {
                bool ready = true;
#pragma unroll
                for (int v = 0; v < DF_WAVES; ++v) ready &= (df_lds_load(&rowslot[rounds - 1][v]) >> 16) == cum;
                if (ready || ++spins > DF_POLL_LIMIT * 16) break;
                __builtin_amdgcn_s_sleep(1);
            }
            df_lds_acquire();
            if (lane == 0) {
                unsigned long long b = best[0];
#pragma unroll
                for (int v = 1; v < DF_WAVES; ++v) b = best[v] > b ? best[v] : b;
                a.cand[wgp] = b;
            }
        }
    }
}

// ---------------------------------------------------------------------------
typedef llm_decode_desc DfHostDesc;
static_assert(sizeof(DfLayer) == sizeof(llm_decode_layer), "DfLayer mirrors llm_decode_layer");

static int df_grid(const DfHostDesc &c, int *n_attn, int *grid) {
    int cus = 0;
    int rc = llm_cu_count_cached(&cus);
    if (rc != LLM_OK) return rc;
    *n_attn = c.n_kv_heads * (c.head_dim >= 128 ? 4 : 1);
    *grid = cus;
    return LLM_OK;
}

static bool df_shapes_ok(const DfHostDesc &c) {
    if (c.n_layers < 1 || c.n_kv_heads <= 0 || c.n_heads % c.n_kv_heads) return false;
    const int G = c.n_heads / c.n_kv_heads, hd = c.head_dim, d = c.d_model, qd = c.n_heads * hd, F = c.ffn_dim;
    if (!((hd == 128 && (G == 1 || G == 4 || G == 8)) || ((hd == 64 || hd == 32) && (G == 1 || G == 4)))) return false;
    if (d % 8 || qd % 8 || F % 8 || c.vocab % 4 || (qd + 2 * c.n_kv_heads * hd) % 4) return false;
    if (d > DF_XS_HALVES || qd > DF_XS_HALVES || F > DF_XS_HALVES) return false;
    if (!rms_shape_ok(d) || d / 4 > WAVE * DF_NORM_R) return false;
    if (c.max_pos <= 0 || c.max_pos % 64) return false;
    return true;
}

template <int HD, int G>
static int df_launch(const DfArgs &a, int grid, hipStream_t s) {
    constexpr int DSN = HD >= 128 ? 4 : 1;
    decode_fused_kernel<HD, G, DSN><<<dim3(grid), dim3(DF_BLOCK), 0, s>>>(a);
    LLM_LAUNCH_CHECK("decode_fused_kernel");
    return LLM_OK;
}

extern "C" {

int llm_decode_fused_supported(const llm_decode_desc *desc) {
    const DfHostDesc &c = *desc;
    if (!df_shapes_ok(c)) return 0;
    int n_attn = 0, grid = 0;
    if (df_grid(c, &n_attn, &grid) != LLM_OK) return 0;
    return grid >= n_attn + 8;
}

// halves in one set of hand-over buffers
size_t llm_decode_fused_ring_halves(const llm_decode_desc *desc) {
    const DfHostDesc &c = *desc;
    const size_t qd = (size_t)c.n_heads * c.head_dim, kvd = (size_t)c.n_kv_heads * c.head_dim;
    return (size_t)c.n_layers * (qd + 2 * kvd + qd + 2 * (size_t)c.d_model + c.ffn_dim);
}

// argmax candidates the LM-head phase leaves in candidates_dev (8 bytes each)
int llm_decode_fused_candidates(const llm_decode_desc *desc) {
    const DfHostDesc &c = *desc;
    int n_attn = 0, grid = 0;
    if (df_grid(c, &n_attn, &grid) != LLM_OK) return 0;
    return grid - n_attn;
}

int llm_decode_fused_phases(const llm_decode_desc *desc) { return 4 * desc->n_layers + 1; }

int llm_decode_fused(const llm_decode_desc *desc, const llm_decode_layer *layers_dev, uint16_t *ring_cur, uint16_t *ring_next, int phase_begin,
                     int phase_end, int32_t *timeouts_dev, llm_stream_t stream) {
    LLM_REQUIRE(desc && layers_dev && ring_cur && ring_next && timeouts_dev, "llm_decode_fused: null pointer");
    const DfHostDesc &c = *desc;
    LLM_REQUIRE(df_shapes_ok(c), "llm_decode_fused: these model shapes are not covered");
    LLM_REQUIRE(ring_cur != ring_next, "llm_decode_fused: a launch cannot re-arm the buffers it uses");
    LLM_REQUIRE(c.rope_table_dev && c.pos_dev && c.tokens_dev && c.embed_dev && c.final_gain_dev && c.lm_head_dev &&
                    c.logits_dev && c.candidates_dev,
                "llm_decode_fused: null pointer in the description");
    const int P = 4 * c.n_layers + 1;
    LLM_REQUIRE(phase_begin >= 0 && phase_begin < phase_end && phase_end <= P, "llm_decode_fused: phases [%d, %d) of %d",
                phase_begin, phase_end, P);
    LLM_REQUIRE(aligned16(ring_cur) && aligned16(ring_next) && aligned16(c.embed_dev) && aligned16(c.lm_head_dev) &&
                    aligned16(c.logits_dev),
                "llm_decode_fused: pointers must be 16-byte aligned");
    int n_attn = 0, grid = 0;
    int rc = df_grid(c, &n_attn, &grid);
    if (rc != LLM_OK) return rc;
    LLM_REQUIRE(grid >= n_attn + 8, "llm_decode_fused: %d CUs for %d attention workgroups", grid, n_attn);
    DfArgs a = {};
    a.layers = (const DfLayer *)layers_dev;
    a.L = c.n_layers;
    a.d = c.d_model;
    a.qd = c.n_heads * c.head_dim;
    a.qkv = a.qd + 2 * c.n_kv_heads * c.head_dim;
    a.F = c.ffn_dim;
    a.vocab = c.vocab;
    a.n_heads = c.n_heads;
    a.n_kv_heads = c.n_kv_heads;
    a.head_dim = c.head_dim;
    a.max_pos = c.max_pos;
    a.eps = c.rms_eps;
    a.rope_table = c.rope_table_dev;
    a.pos_dev = c.pos_dev;
    a.tokens_dev = c.tokens_dev;
    a.embed = (const half_t *)c.embed_dev;
    a.final_gain = (const half_t *)c.final_gain_dev;
    a.lm_head = (const half_t *)c.lm_head_dev;
    a.logits = (half_t *)c.logits_dev;
    a.cand = (unsigned long long *)c.candidates_dev;
    a.ring_cur = ring_cur;
    a.ring_next = ring_next;
    a.timeouts = timeouts_dev;
    a.n_attn = n_attn;
    a.p_begin = phase_begin;
    a.p_end = phase_end;
    hipStream_t s = (hipStream_t)stream;
    const int G = c.n_heads / c.n_kv_heads;
#define DF_CASE(HD_, G_) \
    if (c.head_dim == HD_ && G == G_) return df_launch<HD_, G_>(a, grid, s);
    DF_CASE(128, 4)
    DF_CASE(128, 8)
    DF_CASE(128, 1)
    DF_CASE(64, 4)
    DF_CASE(64, 1)
    DF_CASE(32, 4)
    DF_CASE(32, 1)
#undef DF_CASE
    llm_set_error("llm_decode_fused: head_dim=%d with group size %d is not built", c.head_dim, G);
    return LLM_ERR_INVALID;
}

} // extern "C"
