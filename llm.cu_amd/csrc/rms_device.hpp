// RMSNorm of one row by one workgroup, shared by the standalone kernel and by
// the projection kernels that normalise their input on the way in.
//
// The sum of squares is taken in the order the reference takes it
// (src/inference/inference.cu:309-344): partial i = ((x0^2 + x1^2) + x2^2) + x3^2
// over elements 4i..4i+3, then s[i] += s[i + off] for off = n/2, n/4, ..., 1
// over the n = d/4 partials.  That tree reduces the index bits from the top
// down, so a workgroup of THREADS threads holds slots i = t + THREADS*j in
// thread t, folds j in registers first (the top bits), then the wavefront index
// (every wavefront for itself, from one exchange through LDS) and finishes with
// swaps and shifts between lanes.
// fp32 addition is commutative, so which side of a pair a value sits on does
// not matter; the association is the reference's, hence so are the bits.
#pragma once
#include "common.hpp"

static inline bool rms_shape_ok(int d) {
    if (d <= 0 || d % 4) return false;
    int n = d / 4;
    return (n & (n - 1)) == 0 && n >= 64 && n <= 4096;
}

#define RMS_MAX_R 16 // slots per thread: d/4/THREADS <= 16  (d <= 16384 at 256 threads)

// A thread's share of one row: slot j covers elements 4*(t + THREADS*j)..+3.
template <int MAXR = RMS_MAX_R> struct RmsRow {
    half4_t x[MAXR];
    half4_t g[MAXR];
    int R; // live slots of this thread (0 for spare threads of a narrow row)
};

// Issues the loads of the row (and of the gains when given) and returns at
// once, so the caller can put other loads in flight before rms_finish waits.
template <int THREADS, int MAXR>
__device__ __forceinline__ void rms_load(const half_t *__restrict__ xrow, const half_t *__restrict__ gain, int d,
                                         RmsRow<MAXR> &r) {
    const int t = threadIdx.x;
    const int n = d / 4;
    // fewer slots than threads: the spare threads hold zero slots, which the
    // stride-halving tree folds in without changing any partial sum
    const int R = n >= THREADS ? n / THREADS : 1; // power of two >= 1
    r.R = t < n ? R : 0;
#pragma unroll
    for (int j = 0; j < MAXR; ++j) {
        if (j < r.R) {
            const size_t e = 4 * (size_t)(t + THREADS * j);
            r.x[j] = *reinterpret_cast<const half4_t *>(xrow + e);
            if (gain) r.g[j] = *reinterpret_cast<const half4_t *>(gain + e);
        }
    }
}

// Lane bits 5..0 of the tree, in that order: lane l takes the value of lane l + off for off = 32, 16, 8, 4, 2, 1, so
// lane 0 ends with the reference's association; every lane of the wavefront gets that value.  The two steps
// across 16-lane rows are register swaps (v_permlane32_swap, v_permlane16_swap: both halves of a pair compute
// the same sum, addition being commutative), the four inside a row are DPP row shifts: no trip through LDS.
__device__ __forceinline__ float rms_fold_lanes(float v) {
    uint32_t x = __builtin_bit_cast(uint32_t, v);
    const auto a = __builtin_amdgcn_permlane32_swap(x, x, false, false); // (lo, lo) and (hi, hi)
    v = __builtin_bit_cast(float, (uint32_t)a[0]) + __builtin_bit_cast(float, (uint32_t)a[1]);
    x = __builtin_bit_cast(uint32_t, v);
    const auto b = __builtin_amdgcn_permlane16_swap(x, x, false, false); // rows (0,0,2,2) and (1,1,3,3)
    v = __builtin_bit_cast(float, (uint32_t)b[0]) + __builtin_bit_cast(float, (uint32_t)b[1]);
    v += dpp_move<0x108>(v); // row_shl:8 (lanes shifted in from beyond the row read as 0)
    v += dpp_move<0x104>(v); // row_shl:4
    v += dpp_move<0x102>(v); // row_shl:2
    v += dpp_move<0x101>(v); // row_shl:1
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}

// Sum of squares of the loaded row in the reference's order; every thread gets it.
template <int THREADS, int MAXR>
__device__ __forceinline__ float rms_sum_squares(const RmsRow<MAXR> &r, int d, float *red, const int t = threadIdx.x) {
    const int n = d / 4;
    const int R = n >= THREADS ? n / THREADS : 1;
    float p[MAXR];
#pragma unroll
    for (int j = 0; j < MAXR; ++j) {
        if (j < r.R) {
            const half4_t v = r.x[j];
            float a = (float)v[0], b = (float)v[1], c = (float)v[2], e = (float)v[3];
            p[j] = ((a * a + b * b) + c * c) + e * e;
        } else {
            p[j] = 0.f;
        }
    }
    // top index bits live in j
#pragma unroll
    for (int off = MAXR / 2; off >= 1; off >>= 1) {
        if (off < R) {
#pragma unroll
            for (int j = 0; j < (MAXR > 1 ? MAXR / 2 : 1); ++j)
                if (j < off) p[j] += p[j + off];
        }
    }
    float v = p[0];
    if (THREADS > 64) {
        // thread-index bits above the lane: every wavefront reads the partial of its lane position in each
        // wavefront and folds them top-down itself (one barrier; no wavefront waits for another's fold)
        constexpr int W = THREADS / 64;
        red[t] = v;
        __syncthreads();
        float w[W];
#pragma unroll
        for (int k = 0; k < W; ++k) w[k] = red[(t & 63) + 64 * k];
#pragma unroll
        for (int off = W / 2; off >= 1; off >>= 1) {
#pragma unroll
            for (int k = 0; k < (W > 1 ? W / 2 : 1); ++k)
                if (k < off) w[k] += w[k + off];
        }
        v = w[0];
    }
    return rms_fold_lanes(v);
}

// rms = sqrtf((float)(eps + (double)(ss / d))), the double add as in the
// reference (its eps literal 1e-5 is a double, inference.cu:351).
__device__ __forceinline__ float rms_from_ss(float ss, int d, double eps) {
    return sqrtf((float)(eps + (double)(ss / (float)d)));
}

// y = fp16((x * g) / rms): multiply, then a correctly rounded divide
// (inference.cu:355-358).  dst may be global or LDS memory.
// t: index of the calling thread among the THREADS that share the row (the workgroup's threads by default).
template <int THREADS, int MAXR>
__device__ __forceinline__ void rms_finish(const RmsRow<MAXR> &r, half_t *dst, int d, double eps, float *red,
                                           const int t = threadIdx.x) {
    const float ss = rms_sum_squares<THREADS, MAXR>(r, d, red, t);
    const float rms = rms_from_ss(ss, d, eps);
#pragma unroll
    for (int j = 0; j < MAXR; ++j) {
        if (j < r.R) {
            const size_t e = 4 * (size_t)(t + THREADS * j);
            half4_t o;
#pragma unroll
            for (int k = 0; k < 4; ++k) o[k] = (half_t)(((float)r.x[j][k] * (float)r.g[j][k]) / rms);
            *reinterpret_cast<half4_t *>(dst + e) = o;
        }
    }
}

template <int THREADS>
__device__ __forceinline__ void rms_normalise_row(const half_t *__restrict__ xrow,
                                                  const half_t *__restrict__ gain, half_t *dst, int d,
                                                  double eps, float *red) {
    RmsRow<RMS_MAX_R> r;
    rms_load<THREADS, RMS_MAX_R>(xrow, gain, d, r);
    rms_finish<THREADS, RMS_MAX_R>(r, dst, d, eps, red);
}
