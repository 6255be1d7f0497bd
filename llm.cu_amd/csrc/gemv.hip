// Bandwidth-bound projections for one token (decode): fp16 GEMV with 16-byte
// coalesced, non-temporal weight loads, fp32 accumulation on v_dot2_f32_f16 and
// wavefront reductions.  One kernel covers the plain projection (+ residual),
// the fused SwiGLU pair and the LM head with greedy-argmax candidates, and each
// can take the RMSNorm of its input on the way in.
//
// Layout: w is [N, K] row-major (the reference's [out, in]).  A workgroup of 4
// wavefronts handles 4*rpw rows, four adjacent rows at a time.  Lane l reads
// the 16-byte pieces k = 8l + 512j of a row: every load instruction of a
// wavefront covers a contiguous 1 KiB.  The activation vector (normalised if a
// gain is given) sits in LDS; the first weight loads are issued before it is
// staged so HBM is busy from the first cycle, and loads for the next span are
// in flight while the current one is consumed.
#include <cmath>

#include "common.hpp"
#include "rms_device.hpp"

#define GEMV_THREADS 256
#define GEMV_WAVES 4
#define GEMV_U 4
#define GEMV_SPAN (512 * GEMV_U)
#define GEMV_NORM_R 4 // fused RMSNorm: K <= 4 * 4 * GEMV_THREADS = 4096

// GV_EMBED: GV_PLAIN whose input vector is a row of an embedding table, picked by a token id in device memory
// (the first projection of a decode step: the gather costs no launch of its own).
enum { GV_PLAIN = 0, GV_SWIGLU = 1, GV_LMHEAD = 2, GV_EMBED = 3 };

struct GemvArgs {
    const half_t *x;     // [K]
    const half_t *gain;  // [K] or null: RMSNorm fused into the staging of x
    double eps;
    const half_t *w;     // [N, K]
    const half_t *w2;    // GV_SWIGLU: the up matrix (w is the gate)
    const half_t *res;   // GV_PLAIN: optional residual [N]
    half_t *out;         // [N] (GV_LMHEAD: the fp16 logits)
    unsigned long long *cand; // GV_LMHEAD: one argmax candidate per workgroup
    int N, K, rpw;
    // GV_EMBED: x is the table [vocab, K]; the row is ids[ids_offset ? *ids_offset : 0] (a NaN row for an id outside
    // [0, vocab)), and workgroup 0 leaves a copy of it in x_copy (the residual stream of the layer)
    const int32_t *ids, *ids_offset;
    half_t *x_copy;
    int vocab;
};

// The arguments travel as scalars, the pointers and sizes that the first loads need in front: the file is built
// with kernel-argument preloading, which has the command processor put the first 14 dwords into scalar registers
// before the wavefronts start (a struct passed by value is not preloaded), so the first loads do not wait for a
// trip to the argument buffer.  n_rpw = N | rows per wavefront << 28.
template <int MODE>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_kernel(const half_t *x, const half_t *w, const half_t *gain,
                                                            const half_t *w2, const half_t *res, half_t *out, int n_rpw,
                                                            int K_arg, double eps, unsigned long long *cand,
                                                            const int32_t *ids, const int32_t *ids_offset,
                                                            half_t *x_copy, int vocab) {
    const GemvArgs a = {x,     gain, eps, w, w2, res, out, cand, n_rpw & 0x0fffffff, K_arg, (int)((unsigned)n_rpw >> 28),
                        ids,   ids_offset, x_copy, vocab};
    constexpr int NW = MODE == GV_SWIGLU ? 2 : 1; // weight streams per row
    constexpr bool PLAIN = MODE == GV_PLAIN || MODE == GV_EMBED;
    constexpr int NBUF = 2; // steps in flight per wavefront (2 KB per stream and step)
    extern __shared__ __attribute__((aligned(16))) half_t xs[];
    __shared__ float red[GEMV_THREADS + 1];
    __shared__ unsigned long long best[GEMV_WAVES];
    const int K = a.K, N = a.N;
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    // Row i of wavefront v in workgroup b is i*(4*grid) + 4*b + v: at any moment the
    // whole grid reads one compact, advancing window of the matrix (DRAM pages
    // stay open) instead of one far-apart stream per workgroup.
    const int row_base = blockIdx.x * GEMV_WAVES + wave;
    const int row_step = gridDim.x * GEMV_WAVES;
    const int spr = (K + GEMV_SPAN - 1) / GEMV_SPAN; // spans per row
    const int steps = a.rpw * spr;

    half8_t buf[NBUF][NW][GEMV_U];
    // loads of step s (row i = s / spr, span s % spr) into buf[which]
    auto issue = [&](int which, int i, int sp) {
        int row = row_base + row_step * i;
        row = row < N ? row : N - 1;
        const size_t off = (size_t)row * K + sp * GEMV_SPAN + lane * 8;
#pragma unroll
        for (int u = 0; u < GEMV_U; ++u) {
            const bool ok = sp * GEMV_SPAN + u * 512 + lane * 8 < K;
            buf[which][0][u] = ok ? load8_nt(a.w + off + u * 512) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
            if (NW == 2) buf[which][NW - 1][u] = ok ? load8_nt(a.w2 + off + u * 512) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }
    };

    // cursors: (li, lsp) = next step to load, (i, sp) = step being consumed
    int li = 0, lsp = 0, loaded = 0;
    auto issue_next = [&](int which) {
        if (loaded < steps) {
            issue(which, li, lsp);
            ++loaded;
            if (++lsp == spr) { lsp = 0; ++li; }
        }
    };

    // the activation loads go out first, then NBUF steps of weights; only then
    // does anything wait (the norm's reduction), so HBM is busy throughout
    RmsRow<GEMV_NORM_R> xr;
    constexpr int GEMV_XRAW = 8;
    half8_t xraw[GEMV_XRAW]; // the first GEMV_XRAW * 2048 elements of a plain input vector, asked for before the weights
    if (MODE == GV_EMBED) {
        // the weights do not depend on the token: they go out first, the two dependent loads of the id (position,
        // then id) and the table row follow behind them
#pragma unroll
        for (int b = 0; b < NBUF; ++b) issue_next(b);
        const int id = a.ids[a.ids_offset ? a.ids_offset[0] : 0];
        const bool ok = id >= 0 && id < a.vocab;
        rms_load<GEMV_THREADS, GEMV_NORM_R>(a.x + (size_t)(ok ? id : 0) * K, a.gain, K, xr);
        if (!ok) {
            const half_t nanv = __builtin_bit_cast(half_t, (uint16_t)0x7fffu);
#pragma unroll
            for (int j = 0; j < GEMV_NORM_R; ++j) xr.x[j] = half4_t{nanv, nanv, nanv, nanv};
        }
    } else if (a.gain) {
        rms_load<GEMV_THREADS, GEMV_NORM_R>(a.x, a.gain, K, xr);
    } else {
#pragma unroll
        for (int j = 0; j < GEMV_XRAW; ++j) {
            const int c = (threadIdx.x + GEMV_THREADS * j) * 8;
            if (c < K) xraw[j] = load8(a.x + c);
        }
    }
    if (MODE != GV_EMBED) {
#pragma unroll
        for (int b = 0; b < NBUF; ++b) issue_next(b);
    }
    // the residual of each of this wavefront's rows, asked for now: at the end of a row the value is
    // there instead of one more trip to memory behind the last weight load
    // (four named registers and a select chain below: an array indexed by the row counter would live in
    // scratch memory)
    half_t res0 = (half_t)0.f, res1 = (half_t)0.f, res2 = (half_t)0.f, res3 = (half_t)0.f;
    if (PLAIN && a.res) {
        auto ask = [&](int r) {
            const int row = row_base + row_step * r;
            return (r < a.rpw && row < N) ? a.res[row] : (half_t)0.f;
        };
        res0 = ask(0);
        res1 = ask(1);
        res2 = ask(2);
        res3 = ask(3);
    }
    if (MODE == GV_EMBED || a.gain) {
        rms_finish<GEMV_THREADS, GEMV_NORM_R>(xr, xs, K, a.eps, red);
        if (MODE == GV_EMBED && blockIdx.x == 0) {
#pragma unroll
            for (int j = 0; j < GEMV_NORM_R; ++j)
                if (j < xr.R) *reinterpret_cast<half4_t *>(a.x_copy + 4 * (size_t)(threadIdx.x + GEMV_THREADS * j)) = xr.x[j];
        }
    } else {
#pragma unroll
        for (int j = 0; j < GEMV_XRAW; ++j) {
            const int c = (threadIdx.x + GEMV_THREADS * j) * 8;
            if (c < K) store8(xs + c, xraw[j]);
        }
        for (int c = (threadIdx.x + GEMV_THREADS * GEMV_XRAW) * 8; c < K; c += GEMV_THREADS * 8) store8(xs + c, load8(a.x + c));
    }
    __syncthreads();

    float acc[NW];
#pragma unroll
    for (int j = 0; j < NW; ++j) acc[j] = 0.f;
    unsigned long long mine = 0ull;
    int i = 0, sp = 0;
    auto consume = [&](int which) {
#pragma unroll
        for (int u = 0; u < GEMV_U; ++u) {
            const int k = sp * GEMV_SPAN + u * 512 + lane * 8;
            if (k < K) {
                const half8_t xv = load8(xs + k);
#pragma unroll
                for (int j = 0; j < NW; ++j) acc[j] = dot8(buf[which][j][u], xv, acc[j]);
            }
        }
        if (sp == spr - 1) { // row finished
            const int row = row_base + row_step * i;
            float s0 = wave_sum(acc[0]);
            float s1 = NW == 2 ? wave_sum(acc[NW - 1]) : 0.f;
            if (row < N) {
                if (MODE == GV_SWIGLU) {
                    if (lane == 0) a.out[row] = swiglu_to_half(s0, s1);
                } else if (MODE == GV_LMHEAD) {
                    const half_t h = (half_t)s0;
                    if (lane == 0) a.out[row] = h;
                    const unsigned long long c = pack_candidate(h, row);
                    mine = c > mine ? c : mine;
                } else {
                    if (lane == 0) {
                        half_t hres = (half_t)s0;
                        if (a.res) { // fp16(fp16(sum) + residual), the reference's add_norm on the stored projection
                            const half_t rv = i == 0 ? res0 : i == 1 ? res1 : i == 2 ? res2 : i == 3 ? res3 : a.res[row];
                            hres = (half_t)((float)hres + (float)rv);
                        }
                        a.out[row] = hres;
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < NW; ++j) acc[j] = 0.f;
        }
        if (++sp == spr) { sp = 0; ++i; }
    };
    // NBUF steps per trip: each register buffer is refilled right after it is consumed
    for (int s = 0; s < steps; s += NBUF) {
#pragma unroll
        for (int b = 0; b < NBUF; ++b) {
            if (s + b < steps) {
                consume(b);
                issue_next(b);
            }
        }
    }
    if (MODE == GV_LMHEAD) {
        if (lane == 0) best[wave] = mine;
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned long long b = best[0];
#pragma unroll
            for (int v = 1; v < GEMV_WAVES; ++v) b = best[v] > b ? best[v] : b;
            a.cand[blockIdx.x] = b;
        }
    }
}

// candidates over plain fp16 values (argmax alone)
// (blockIdx.y: row of a [rows, ld] matrix; its candidates follow those of the rows before it)
__global__ __launch_bounds__(256) void argmax_candidates_kernel(const half_t *__restrict__ v, int n,
                                                                unsigned long long *__restrict__ cand, int ld) {
    __shared__ unsigned long long best[256];
    unsigned long long mine = 0ull;
    v += (size_t)blockIdx.y * ld;
    cand += (size_t)blockIdx.y * gridDim.x;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        unsigned long long c = pack_candidate(v[i], i);
        mine = c > mine ? c : mine;
    }
    best[threadIdx.x] = mine;
    __syncthreads();
    for (int off = 128; off >= 1; off >>= 1) {
        if ((int)threadIdx.x < off && best[threadIdx.x + off] > best[threadIdx.x]) best[threadIdx.x] = best[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) cand[blockIdx.x] = best[0];
}

// Final pick: one block folds the candidates; optionally feeds the next step.
__global__ __launch_bounds__(1024) void argmax_final_kernel(const unsigned long long *__restrict__ cand, int n,
                                                            int32_t *__restrict__ token,
                                                            int32_t *__restrict__ tokens,
                                                            int32_t *__restrict__ pos) {
    __shared__ unsigned long long best[1024];
    unsigned long long mine = 0ull;
    cand += (size_t)blockIdx.x * n; // one block per row
    token += blockIdx.x;
    for (int i = threadIdx.x; i < n; i += 1024) mine = cand[i] > mine ? cand[i] : mine;
    best[threadIdx.x] = mine;
    __syncthreads();
    for (int off = 512; off >= 1; off >>= 1) {
        if ((int)threadIdx.x < off && best[threadIdx.x + off] > best[threadIdx.x]) best[threadIdx.x] = best[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        unsigned long long b = best[0];
        int tok = b == 0ull ? 0 : (int)(0xffffffffu - (uint32_t)(b & 0xffffffffull));
        token[0] = tok;
        if (tokens && pos) {
            int p = pos[0];
            tokens[p + 1] = tok;
            pos[0] = p + 1;
        }
    }
}

// ---------------------------------------------------------------------------
// Rows per wavefront, from sweeps on MI355X at the LLaMA3-8B shapes: many small
// workgroups win (the hardware keeps refilling CUs as wavefronts retire); only
// the norm-fused QKV projection and the 128K-row LM head amortise their
// per-workgroup prologue over more than one row.
static int rows_per_wave(int mode, int N, bool norm) {
    if (mode == GV_LMHEAD) return N >= 32768 ? 3 : 1;
    if ((mode == GV_PLAIN || mode == GV_EMBED) && norm && N >= 6144) return 2;
    return 1;
}

static int gemv_blocks(int N, int rpw) { return (N + GEMV_WAVES * rpw - 1) / (GEMV_WAVES * rpw); }

template <int MODE> static int gemv_dispatch(GemvArgs a, hipStream_t s) {
    const size_t smem = (size_t)a.K * sizeof(half_t);
    LLM_REQUIRE(a.K % 8 == 0 && smem <= 56 * 1024, "GEMV: K=%d must be a multiple of 8 and fit 56 KiB of LDS", a.K);
    LLM_REQUIRE(MODE != GV_EMBED || (a.gain && a.ids && a.x_copy && a.vocab > 0), "GEMV on an embedding row: gain, ids, copy, vocab");
    LLM_REQUIRE(!a.gain || (rms_shape_ok(a.K) && a.K <= 4 * GEMV_NORM_R * GEMV_THREADS),
                "GEMV with RMSNorm: K=%d (need K/4 a power of two in [64, %d])", a.K, GEMV_NORM_R * GEMV_THREADS);
    LLM_REQUIRE(a.N < (1 << 28) && a.rpw >= 1 && a.rpw < 16, "GEMV: N=%d rows per wavefront %d", a.N, a.rpw);
    gemv_kernel<MODE><<<dim3(gemv_blocks(a.N, a.rpw)), dim3(GEMV_THREADS), smem, s>>>(a.x, a.w, a.gain, a.w2, a.res, a.out,
                                                                                     a.N | (a.rpw << 28), a.K, a.eps, a.cand,
                                                                                     a.ids, a.ids_offset, a.x_copy, a.vocab);
    LLM_LAUNCH_CHECK("gemv_kernel");
    return LLM_OK;
}

int gemv_launch(const half_t *x, const half_t *gain, double eps, const half_t *w, const half_t *res, half_t *out,
                int N, int K, hipStream_t s) {
    GemvArgs a = {x, gain, eps, w, nullptr, res, out, nullptr, N, K, rows_per_wave(GV_PLAIN, N, gain != nullptr)};
    return gemv_dispatch<GV_PLAIN>(a, s);
}

int gemv_embed_launch(const half_t *table, const int32_t *ids, const int32_t *ids_offset, int vocab, half_t *x_copy,
                      const half_t *gain, double eps, const half_t *w, half_t *out, int N, int K, hipStream_t s) {
    GemvArgs a = {table, gain, eps, w, nullptr, nullptr, out, nullptr, N, K, rows_per_wave(GV_EMBED, N, true),
                  ids,   ids_offset, x_copy, vocab};
    return gemv_dispatch<GV_EMBED>(a, s);
}

int gemv_swiglu_launch(const half_t *x, const half_t *gain, double eps, const half_t *wg, const half_t *wu,
                       half_t *out, int N, int K, hipStream_t s) {
    GemvArgs a = {x, gain, eps, wg, wu, nullptr, out, nullptr, N, K, rows_per_wave(GV_SWIGLU, N, gain != nullptr)};
    return gemv_dispatch<GV_SWIGLU>(a, s);
}

extern "C" {

size_t llm_lmhead_workspace_bytes(int vocab) {
    size_t blocks = (size_t)gemv_blocks(vocab, 1); // upper bound for any rows-per-wave choice
    if (blocks < 1024) blocks = 1024;
    return blocks * sizeof(unsigned long long);
}

int llm_norm_lmhead_argmax(const uint16_t *x, const uint16_t *gain, double eps, const uint16_t *w, uint16_t *logits,
                           int32_t *token, int32_t *tokens, int32_t *pos, int vocab, int K, void *workspace,
                           llm_stream_t stream) {
    LLM_REQUIRE(x && w && logits && token && workspace, "llm_lmhead_argmax: null pointer");
    LLM_REQUIRE(vocab > 0 && K > 0, "llm_lmhead_argmax: vocab=%d K=%d", vocab, K);
    LLM_REQUIRE(aligned16(x) && aligned16(w) && (!gain || aligned16(gain)), "llm_lmhead_argmax: pointers must be 16-byte aligned");
    LLM_REQUIRE((tokens == nullptr) == (pos == nullptr), "llm_lmhead_argmax: tokens and pos go together");
    hipStream_t s = (hipStream_t)stream;
    const int rpw = rows_per_wave(GV_LMHEAD, vocab, gain != nullptr);
    GemvArgs a = {(const half_t *)x, (const half_t *)gain, eps, (const half_t *)w, nullptr, nullptr, (half_t *)logits,
                  (unsigned long long *)workspace, vocab, K, rpw};
    int rc = gemv_dispatch<GV_LMHEAD>(a, s);
    if (rc != LLM_OK) return rc;
    argmax_final_kernel<<<dim3(1), dim3(1024), 0, s>>>((const unsigned long long *)workspace, gemv_blocks(vocab, rpw),
                                                       token, tokens, pos);
    LLM_LAUNCH_CHECK("argmax_final_kernel");
    return LLM_OK;
}

int llm_lmhead_argmax(const uint16_t *x, const uint16_t *w, uint16_t *logits, int32_t *token, int32_t *tokens,
                      int32_t *pos, int vocab, int K, void *workspace, llm_stream_t stream) {
    return llm_norm_lmhead_argmax(x, nullptr, 0.0, w, logits, token, tokens, pos, vocab, K, workspace, stream);
}

int llm_argmax_f16_rows(const uint16_t *logits, int ld, int rows, int n, int32_t *tokens, void *workspace,
                        llm_stream_t stream) {
    LLM_REQUIRE(logits && tokens && workspace, "llm_argmax_f16: null pointer");
    LLM_REQUIRE(n > 0 && rows > 0 && rows <= 65535 && ld >= n, "llm_argmax_f16: rows=%d n=%d ld=%d", rows, n, ld);
    hipStream_t s = (hipStream_t)stream;
    int blocks = (n + 255) / 256;
    if (blocks > 1024) blocks = 1024;
    argmax_candidates_kernel<<<dim3(blocks, rows), dim3(256), 0, s>>>((const half_t *)logits, n,
                                                                      (unsigned long long *)workspace, ld);
    LLM_LAUNCH_CHECK("argmax_candidates_kernel");
    argmax_final_kernel<<<dim3(rows), dim3(1024), 0, s>>>((const unsigned long long *)workspace, blocks, tokens, nullptr,
                                                          nullptr);
    LLM_LAUNCH_CHECK("argmax_final_kernel");
    return LLM_OK;
}

int llm_argmax_f16(const uint16_t *logits, int n, int32_t *token, void *workspace, llm_stream_t stream) {
    return llm_argmax_f16_rows(logits, n, 1, n, token, workspace, stream);
}

} // extern "C"
