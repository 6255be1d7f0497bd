// Bandwidth-bound projections for one token (decode): fp16 GEMV with 16-byte
// coalesced weight loads, fp32 accumulation on v_dot2_f32_f16, wavefront
// reductions; plus the fused SwiGLU pair and the LM head with greedy argmax.
//
// Layout: w is [N, K] row-major (the reference's [out, in]).  One wavefront
// owns R consecutive rows at a time; lane l streams 16-byte pieces
// k = 8l + 512j of each row, so a wavefront reads whole contiguous 1 KiB
// spans of a row per load.  The activation vector sits in LDS.
#include <cmath>

#include "common.hpp"

#define GEMV_THREADS 256
#define GEMV_WAVES 4

__device__ __forceinline__ void stage_x(const half_t *__restrict__ x, half_t *xs, int K) {
    for (int c = threadIdx.x * 8; c < K; c += GEMV_THREADS * 8) store8(xs + c, load8(x + c));
    __syncthreads();
}

// Accumulates R rows against xs; U independent 16-byte loads per row in flight.
template <int R, int U>
__device__ __forceinline__ void gemv_rows(const half_t *const (&wp)[R], const half_t *xs, int K, int lane,
                                          float (&acc)[R]) {
    const int span = 512 * U;
    const int kmain = K / span * span;
    for (int k0 = 0; k0 < kmain; k0 += span) {
        half8_t wv[R][U];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int u = 0; u < U; ++u) wv[r][u] = load8(wp[r] + k0 + u * 512 + lane * 8);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            half8_t xv = load8(xs + k0 + u * 512 + lane * 8);
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = dot8(wv[r][u], xv, acc[r]);
        }
    }
    for (int k = kmain + lane * 8; k < K; k += 512) {
        half8_t xv = load8(xs + k);
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = dot8(load8(wp[r] + k), xv, acc[r]);
    }
}

template <int R, int U>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_kernel(const half_t *__restrict__ x,
                                                            const half_t *__restrict__ w,
                                                            const half_t *__restrict__ res,
                                                            half_t *__restrict__ out, int N, int K) {
    extern __shared__ half_t xs[];
    stage_x(x, xs, K);
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int row0 = (blockIdx.x * GEMV_WAVES + wave) * R;
    if (row0 >= N) return;
    const half_t *wp[R];
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int row = row0 + r < N ? row0 + r : N - 1;
        wp[r] = w + (size_t)row * K;
        acc[r] = 0.f;
    }
    gemv_rows<R, U>(wp, xs, K, lane, acc);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        float s = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) out[row0 + r] = finish(s, res ? res + row0 + r : nullptr);
    }
}

__device__ __forceinline__ float silu_f(float g) { return g / (1.0f + expf(-g)); }

template <int R, int U>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_swiglu_kernel(const half_t *__restrict__ x,
                                                                   const half_t *__restrict__ wg,
                                                                   const half_t *__restrict__ wu,
                                                                   half_t *__restrict__ out, int N, int K) {
    extern __shared__ half_t xs[];
    stage_x(x, xs, K);
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int row0 = (blockIdx.x * GEMV_WAVES + wave) * R;
    if (row0 >= N) return;
    const half_t *wp[2 * R];
    float acc[2 * R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int row = row0 + r < N ? row0 + r : N - 1;
        wp[r] = wg + (size_t)row * K;
        wp[R + r] = wu + (size_t)row * K;
        acc[r] = acc[R + r] = 0.f;
    }
    gemv_rows<2 * R, U>(wp, xs, K, lane, acc);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        float g = wave_sum(acc[r]);
        float u = wave_sum(acc[R + r]);
        if (lane == 0 && row0 + r < N) out[row0 + r] = (half_t)(silu_f(g) * u);
    }
}

// LM head: logits for R rows per wavefront plus a per-block argmax candidate.
// Candidates are packed (order key + 1) << 32 | ~index so that an unsigned
// max picks the largest logit and, among equals, the lowest index; NaN packs
// to 0 and never wins.
__device__ __forceinline__ unsigned long long pack_candidate(half_t h, int idx) {
    uint16_t bits = __builtin_bit_cast(uint16_t, h);
    if ((bits & 0x7fffu) > 0x7c00u) return 0ull;
    return ((unsigned long long)(f16_order_key(bits) + 1u) << 32) | (unsigned long long)(0xffffffffu - (uint32_t)idx);
}

template <int R, int U>
__global__ __launch_bounds__(GEMV_THREADS) void lmhead_kernel(const half_t *__restrict__ x,
                                                              const half_t *__restrict__ w,
                                                              half_t *__restrict__ logits,
                                                              unsigned long long *__restrict__ cand, int N,
                                                              int K) {
    extern __shared__ half_t xs[];
    __shared__ unsigned long long best[GEMV_WAVES];
    stage_x(x, xs, K);
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int row0 = (blockIdx.x * GEMV_WAVES + wave) * R;
    unsigned long long mine = 0ull;
    if (row0 < N) {
        const half_t *wp[R];
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int row = row0 + r < N ? row0 + r : N - 1;
            wp[r] = w + (size_t)row * K;
            acc[r] = 0.f;
        }
        gemv_rows<R, U>(wp, xs, K, lane, acc);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float s = wave_sum(acc[r]);
            if (row0 + r < N) {
                half_t h = (half_t)s;
                if (lane == 0) logits[row0 + r] = h;
                unsigned long long c = pack_candidate(h, row0 + r);
                mine = c > mine ? c : mine;
            }
        }
    }
    if (lane == 0) best[wave] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long b = best[0];
#pragma unroll
        for (int i = 1; i < GEMV_WAVES; ++i) b = best[i] > b ? best[i] : b;
        cand[blockIdx.x] = b;
    }
}

// candidates over plain fp16 values (argmax alone)
__global__ __launch_bounds__(256) void argmax_candidates_kernel(const half_t *__restrict__ v, int n,
                                                                unsigned long long *__restrict__ cand) {
    __shared__ unsigned long long best[256];
    unsigned long long mine = 0ull;
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
int gemv_launch(const half_t *x, const half_t *w, const half_t *res, half_t *out, int N, int K, hipStream_t s) {
    const size_t smem = (size_t)K * sizeof(half_t);
    LLM_REQUIRE(smem <= 64 * 1024, "GEMV: K=%d does not fit the 64 KiB LDS staging", K);
    constexpr int R = 2, U = 4;
    const int blocks = (N + GEMV_WAVES * R - 1) / (GEMV_WAVES * R);
    gemv_kernel<R, U><<<dim3(blocks), dim3(GEMV_THREADS), smem, s>>>(x, w, res, out, N, K);
    LLM_LAUNCH_CHECK("gemv_kernel");
    return LLM_OK;
}

int gemv_swiglu_launch(const half_t *x, const half_t *wg, const half_t *wu, half_t *out, int N, int K,
                       hipStream_t s) {
    const size_t smem = (size_t)K * sizeof(half_t);
    LLM_REQUIRE(smem <= 64 * 1024, "GEMV: K=%d does not fit the 64 KiB LDS staging", K);
    constexpr int R = 1, U = 4;
    const int blocks = (N + GEMV_WAVES * R - 1) / (GEMV_WAVES * R);
    gemv_swiglu_kernel<R, U><<<dim3(blocks), dim3(GEMV_THREADS), smem, s>>>(x, wg, wu, out, N, K);
    LLM_LAUNCH_CHECK("gemv_swiglu_kernel");
    return LLM_OK;
}

extern "C" {

size_t llm_lmhead_workspace_bytes(int vocab) {
    constexpr int R = 2;
    size_t blocks = ((size_t)vocab + GEMV_WAVES * R - 1) / (GEMV_WAVES * R);
    if (blocks < 1024) blocks = 1024;
    return blocks * sizeof(unsigned long long);
}

int llm_lmhead_argmax(const uint16_t *x, const uint16_t *w, uint16_t *logits, int32_t *token, int32_t *tokens,
                      int32_t *pos, int vocab, int K, void *workspace, llm_stream_t stream) {
    LLM_REQUIRE(x && w && logits && token && workspace, "llm_lmhead_argmax: null pointer");
    LLM_REQUIRE(vocab > 0 && K > 0 && K % 8 == 0, "llm_lmhead_argmax: vocab=%d K=%d", vocab, K);
    LLM_REQUIRE(aligned16(x) && aligned16(w), "llm_lmhead_argmax: pointers must be 16-byte aligned");
    LLM_REQUIRE((tokens == nullptr) == (pos == nullptr), "llm_lmhead_argmax: tokens and pos go together");
    const size_t smem = (size_t)K * sizeof(half_t);
    LLM_REQUIRE(smem <= 64 * 1024, "llm_lmhead_argmax: K=%d does not fit the LDS staging", K);
    constexpr int R = 2, U = 4;
    const int blocks = (vocab + GEMV_WAVES * R - 1) / (GEMV_WAVES * R);
    hipStream_t s = (hipStream_t)stream;
    lmhead_kernel<R, U><<<dim3(blocks), dim3(GEMV_THREADS), smem, s>>>(
        (const half_t *)x, (const half_t *)w, (half_t *)logits, (unsigned long long *)workspace, vocab, K);
    LLM_LAUNCH_CHECK("lmhead_kernel");
    argmax_final_kernel<<<dim3(1), dim3(1024), 0, s>>>((const unsigned long long *)workspace, blocks, token, tokens,
                                                       pos);
    LLM_LAUNCH_CHECK("argmax_final_kernel");
    return LLM_OK;
}

int llm_argmax_f16(const uint16_t *logits, int n, int32_t *token, void *workspace, llm_stream_t stream) {
    LLM_REQUIRE(logits && token && workspace, "llm_argmax_f16: null pointer");
    LLM_REQUIRE(n > 0, "llm_argmax_f16: n=%d", n);
    hipStream_t s = (hipStream_t)stream;
    int blocks = (n + 255) / 256;
    if (blocks > 1024) blocks = 1024;
    argmax_candidates_kernel<<<dim3(blocks), dim3(256), 0, s>>>((const half_t *)logits, n,
                                                                (unsigned long long *)workspace);
    LLM_LAUNCH_CHECK("argmax_candidates_kernel");
    argmax_final_kernel<<<dim3(1), dim3(1024), 0, s>>>((const unsigned long long *)workspace, blocks, token, nullptr,
                                                       nullptr);
    LLM_LAUNCH_CHECK("argmax_final_kernel");
    return LLM_OK;
}

} // extern "C"
