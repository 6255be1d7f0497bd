// Shared device/host helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "llmcu_hip.h"

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

#define WAVE 64

// ---- error plumbing -------------------------------------------------------
void llm_set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

#define LLM_HIP_CHECK(expr)                                                          \
    do {                                                                             \
        hipError_t _e = (expr);                                                      \
        if (_e != hipSuccess) {                                                      \
            llm_set_error("%s: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
            return LLM_ERR_HIP;                                                      \
        }                                                                            \
    } while (0)

#define LLM_REQUIRE(cond, ...)            \
    do {                                  \
        if (!(cond)) {                    \
            llm_set_error(__VA_ARGS__);   \
            return LLM_ERR_INVALID;       \
        }                                 \
    } while (0)

// Launch check: hipGetLastError right after the <<<>>>.
#define LLM_LAUNCH_CHECK(name)                                                      \
    do {                                                                            \
        hipError_t _e = hipGetLastError();                                          \
        if (_e != hipSuccess) {                                                     \
            llm_set_error("launch of %s: %s", name, hipGetErrorString(_e));         \
            return LLM_ERR_HIP;                                                     \
        }                                                                           \
    } while (0)

// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per device for one kernel instantiation.
// `done` is that instantiation's bit mask of devices already set; two threads racing on a fresh device
// both set the same value, which is harmless.
static inline int llm_ensure_max_smem(const void *kern, size_t smem, std::atomic<uint64_t> &done) {
    int dev = 0;
    LLM_HIP_CHECK(hipGetDevice(&dev));
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return LLM_OK;
    LLM_HIP_CHECK(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    done.fetch_or(bit, std::memory_order_release);
    return LLM_OK;
}

// Compute units of the current device (looked up once per device).
static inline int llm_cu_count_cached(int *cus) {
    static std::atomic<int> cache[64];
    int dev = 0;
    LLM_HIP_CHECK(hipGetDevice(&dev));
    int n = cache[dev & 63].load(std::memory_order_relaxed);
    if (n == 0) {
        LLM_HIP_CHECK(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev));
        cache[dev & 63].store(n, std::memory_order_relaxed);
    }
    *cus = n;
    return LLM_OK;
}

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- device helpers ---------------------------------------------------------
// Cross-lane moves inside a row of 16 lanes run on the VALU's DPP path (no trip
// through the LDS crossbar that __shfl uses).  Controls: quad_perm(1,0,3,2),
// quad_perm(2,3,0,1), row_half_mirror, row_mirror.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// Sum over aligned groups of N lanes (N = 2, 4, 8 or 16); every lane of the group gets it.
template <int N> __device__ __forceinline__ float group_sum(float v) {
    static_assert(N == 1 || N == 2 || N == 4 || N == 8 || N == 16, "group size");
    if (N >= 2) v += dpp_move<0xB1>(v);
    if (N >= 4) v += dpp_move<0x4E>(v);
    if (N >= 8) v += dpp_move<0x141>(v);
    if (N >= 16) v += dpp_move<0x140>(v);
    return v;
}

template <int N> __device__ __forceinline__ float group_max(float v) {
    if (N >= 2) v = fmaxf(v, dpp_move<0xB1>(v));
    if (N >= 4) v = fmaxf(v, dpp_move<0x4E>(v));
    if (N >= 8) v = fmaxf(v, dpp_move<0x141>(v));
    if (N >= 16) v = fmaxf(v, dpp_move<0x140>(v));
    return v;
}

// max / sum over the lanes l, l ^ 16, l ^ 32, l ^ 48 (one lane of each 16-lane row); every lane gets the result.
// Two swaps between rows (v_permlane16_swap, v_permlane32_swap) instead of two trips through the LDS crossbar
// (ds_bpermute); the operands meet in the same order as with __shfl_xor(v, 16) followed by __shfl_xor(v, 32).
__device__ __forceinline__ float rows_max(float v) {
    uint32_t x = __builtin_bit_cast(uint32_t, v);
    const auto a = __builtin_amdgcn_permlane16_swap(x, x, false, false); // rows (0,0,2,2) and (1,1,3,3)
    v = fmaxf(__builtin_bit_cast(float, (uint32_t)a[0]), __builtin_bit_cast(float, (uint32_t)a[1]));
    x = __builtin_bit_cast(uint32_t, v);
    const auto b = __builtin_amdgcn_permlane32_swap(x, x, false, false); // halves (lo,lo) and (hi,hi)
    return fmaxf(__builtin_bit_cast(float, (uint32_t)b[0]), __builtin_bit_cast(float, (uint32_t)b[1]));
}
__device__ __forceinline__ float rows_sum(float v) {
    uint32_t x = __builtin_bit_cast(uint32_t, v);
    const auto a = __builtin_amdgcn_permlane16_swap(x, x, false, false);
    v = __builtin_bit_cast(float, (uint32_t)a[0]) + __builtin_bit_cast(float, (uint32_t)a[1]);
    x = __builtin_bit_cast(uint32_t, v);
    const auto b = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return __builtin_bit_cast(float, (uint32_t)b[0]) + __builtin_bit_cast(float, (uint32_t)b[1]);
}

__device__ __forceinline__ float wave_sum(float v) { return rows_sum(group_sum<16>(v)); }

__device__ __forceinline__ float wave_max(float v) { return rows_max(group_max<16>(v)); }

// 8 fp16 x 8 fp16 -> fp32, accumulated with v_dot2_f32_f16.
__device__ __forceinline__ float dot8(half8_t a, half8_t b, float acc) {
    acc = __builtin_amdgcn_fdot2(half2_t{a[0], a[1]}, half2_t{b[0], b[1]}, acc, false);
    acc = __builtin_amdgcn_fdot2(half2_t{a[2], a[3]}, half2_t{b[2], b[3]}, acc, false);
    acc = __builtin_amdgcn_fdot2(half2_t{a[4], a[5]}, half2_t{b[4], b[5]}, acc, false);
    acc = __builtin_amdgcn_fdot2(half2_t{a[6], a[7]}, half2_t{b[6], b[7]}, acc, false);
    return acc;
}

__device__ __forceinline__ half8_t load8(const half_t *p) { return *reinterpret_cast<const half8_t *>(p); }
// streamed once: do not keep the line in the caches
__device__ __forceinline__ half8_t load8_nt(const half_t *p) {
    uint4_t v = __builtin_nontemporal_load(reinterpret_cast<const uint4_t *>(p));
    return __builtin_bit_cast(half8_t, v);
}
__device__ __forceinline__ void store8(half_t *p, half8_t v) { *reinterpret_cast<half8_t *>(p) = v; }

// RoPE of four adjacent pairs (8 halves): (e, o) -> (c e - s o, s e + c o) with unfused multiplies (the device code
// is compiled with -ffp-contract=off), each result rounded to fp16.  cs: the four (cos, sin) pairs of the position.
__device__ __forceinline__ half8_t rope_rotate8(half8_t v, const float *__restrict__ cs) {
    half8_t o;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const float c = cs[2 * p], s = cs[2 * p + 1];
        const float e = (float)v[2 * p], od = (float)v[2 * p + 1];
        const float ce = c * e, so = s * od, se = s * e, co = c * od;
        o[2 * p] = (half_t)(ce - so);
        o[2 * p + 1] = (half_t)(se + co);
    }
    return o;
}

// fp16 result with an optional residual: the reference stores the projection
// as fp16 and then adds the fp16 residual in fp32 (two roundings).
__device__ __forceinline__ half_t finish(float acc, const half_t *res) {
    half_t h = (half_t)acc;
    if (res) h = (half_t)((float)h + (float)*res);
    return h;
}

// Bit pattern of the fp16 logit mapped to an unsigned key that orders like
// the value (NaN excluded by the caller): used by the argmax reductions.
__device__ __forceinline__ uint32_t f16_order_key(uint16_t bits) {
    // -0 and +0 must compare equal: map -0 to +0 first.
    if (bits == 0x8000u) bits = 0;
    return (bits & 0x8000u) ? (uint32_t)(0x7fffu - (bits & 0x7fffu)) : (uint32_t)(0x8000u + bits);
}

// SiLU (src/inference/inference.cu:451-453: x / (1 + expf(-x)) in fp32).  The reference's expf is CUDA's, whose bits
// no other math library reproduces, so this is a floating-point step inside the stated tolerance either way: the
// hardware exponential and reciprocal (a few fp32 ulp, three orders of magnitude below the fp16 rounding that
// follows) instead of the library expf and the IEEE division, which cost 2 % of the prompt pass's gate/up GEMM.
// Every path (GEMV, skinny, GEMM, fused decode) goes through this one function.
__device__ __forceinline__ float silu_f(float g) { return __fdividef(g, 1.0f + __expf(-g)); }

// fp16(SiLU(gate) * up) as the reference rounds it (src/inference/inference.cu:513-516: the product is an
// fp32 value, then __float2half): the empty asm keeps the compiler from folding the multiply and the
// conversion into one instruction that rounds the exact product once (v_fma_mixlo_f16), which differs
// from the reference's two roundings in the last bit now and then.
__device__ __forceinline__ half_t swiglu_to_half(float gate, float up) {
    float p = silu_f(gate) * up;
    asm volatile("" : "+v"(p));
    return (half_t)p;
}

// Candidates are packed (order key + 1) << 32 | ~index so that an unsigned max
// picks the largest logit and, among equals, the lowest index; NaN packs to 0
// and never wins.
__device__ __forceinline__ unsigned long long pack_candidate(half_t h, int idx) {
    uint16_t bits = __builtin_bit_cast(uint16_t, h);
    if ((bits & 0x7fffu) > 0x7c00u) return 0ull;
    return ((unsigned long long)(f16_order_key(bits) + 1u) << 32) | (unsigned long long)(0xffffffffu - (uint32_t)idx);
}
