// RMSNorm of one row by one workgroup, shared by the standalone kernel and by
// the projection kernels that normalise their input on the way in.
//
// The sum of squares is taken in the order the reference takes it
// (src/inference/inference.cu:309-344): partial i = ((x0^2 + x1^2) + x2^2) + x3^2
// over elements 4i..4i+3, then s[i] += s[i + off] for off = n/2, n/4, ..., 1
// over the n = d/4 partials.  That tree reduces the index bits from the top
// down, so a workgroup of THREADS threads holds slots i = t + THREADS*j in
// thread t, folds j in registers first (the top bits), then folds the thread
// index through LDS down to one wavefront and finishes with lane shuffles.
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

// Returns ss for the row; every thread gets the value.  `vals` receives the
// thread's 4*R input elements (slot j at vals[4j..4j+3]).
template <int THREADS>
__device__ __forceinline__ float rms_sum_squares(const half_t *__restrict__ xrow, int d, float *red,
                                                 half4_t *vals, int &R_out) {
    const int t = threadIdx.x;
    const int n = d / 4;
    const int R = n / THREADS; // power of two >= 1
    R_out = R;
    float p[RMS_MAX_R];
#pragma unroll
    for (int j = 0; j < RMS_MAX_R; ++j) {
        if (j < R) {
            half4_t v = *reinterpret_cast<const half4_t *>(xrow + 4 * (size_t)(t + THREADS * j));
            vals[j] = v;
            float a = (float)v[0], b = (float)v[1], c = (float)v[2], e = (float)v[3];
            p[j] = ((a * a + b * b) + c * c) + e * e;
        } else {
            p[j] = 0.f;
        }
    }
    // top index bits live in j
#pragma unroll
    for (int off = RMS_MAX_R / 2; off >= 1; off >>= 1) {
        if (off < R) {
#pragma unroll
            for (int j = 0; j < RMS_MAX_R / 2; ++j)
                if (j < off) p[j] += p[j + off];
        }
    }
    float v = p[0];
    if (THREADS > 64) {
        red[t] = v;
        __syncthreads();
        for (int off = THREADS / 2; off >= 64; off >>= 1) {
            if (t < off) red[t] += red[t + off];
            __syncthreads();
        }
        v = red[t & 63]; // wave 0 holds the live values; other waves read them too (unused)
    }
    // lane bits 5..0, in that order; lane 0 of wave 0 ends with the reference's sum
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_down(v, off);
    if (THREADS > 64) {
        __syncthreads();
        if (t == 0) red[THREADS] = v;
        __syncthreads();
        v = red[THREADS];
    } else {
        v = __shfl(v, 0);
    }
    return v;
}

// rms = sqrtf((float)(eps + (double)(ss / d))), the double add as in the
// reference (its eps literal 1e-5 is a double, inference.cu:351).
__device__ __forceinline__ float rms_from_ss(float ss, int d, double eps) {
    return sqrtf((float)(eps + (double)(ss / (float)d)));
}

// y = fp16((x * g) / rms): multiply, then a correctly rounded divide
// (inference.cu:355-358).  dst may be global or LDS memory.
template <int THREADS>
__device__ __forceinline__ void rms_normalise_row(const half_t *__restrict__ xrow,
                                                  const half_t *__restrict__ gain, half_t *dst, int d,
                                                  double eps, float *red) {
    half4_t vals[RMS_MAX_R];
    int R;
    float ss = rms_sum_squares<THREADS>(xrow, d, red, vals, R);
    float rms = rms_from_ss(ss, d, eps);
    const int t = threadIdx.x;
#pragma unroll
    for (int j = 0; j < RMS_MAX_R; ++j) {
        if (j < R) {
            const size_t e = 4 * (size_t)(t + THREADS * j);
            half4_t g = *reinterpret_cast<const half4_t *>(gain + e);
            half4_t o;
#pragma unroll
            for (int k = 0; k < 4; ++k) o[k] = (half_t)(((float)vals[j][k] * (float)g[k]) / rms);
            *reinterpret_cast<half4_t *>(dst + e) = o;
        }
    }
}
