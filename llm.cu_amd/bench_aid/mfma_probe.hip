// Measurement aid, not part of the token loop: what the matrix pipes of this part sustain when nothing but
// MFMAs run, with operands of a chosen kind.  The dense fp16 peak (2.5 PFLOP/s) assumes the full clock; under the
// board's power limit the sustained rate depends on how many operand bits toggle, so the ceiling that the
// prompt-pass GEMMs can be held against is this probe's figure for operands distributed like theirs.
#include <hip/hip_runtime.h>

#include "common.hpp"

// Every wavefront: `iters` rounds of MFMAs over four A and four B operand sets (every MFMA sees operands that
// differ from its predecessor's, as in a GEMM) into 128 accumulator registers (no dependency stalls): sixteen
// v_mfma_f32_32x32x16_f16 into eight accumulators, or (SMALL) thirty-two v_mfma_f32_16x16x32_f16 into
// thirty-two -- the same flops per round.  kind bit 0 clear: all operands 1.0; set: normal(0, 1) activations
// against normal(0, 0.02) weights from a counter-based generator, different in every lane and set.
template <bool SMALL> __global__ __launch_bounds__(256) void mfma_probe_kernel(float *sink, int iters, int kind) {
    half8_t a[4], b[4];
    const unsigned id = blockIdx.x * blockDim.x + threadIdx.x;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if ((kind & 1) == 0) {
                a[p][i] = (half_t)1.0f;
                b[p][i] = (half_t)1.0f;
            } else {
                // two hashes -> Box-Muller
                unsigned h1 = (id * 32u + p * 8u + i) * 2654435761u + 12345u, h2 = h1 * 1664525u + 1013904223u;
                h1 ^= h1 >> 15, h1 *= 2246822519u, h1 ^= h1 >> 13;
                h2 ^= h2 >> 16, h2 *= 3266489917u, h2 ^= h2 >> 15;
                const float u1 = ((h1 >> 8) + 1) * (1.0f / 16777217.0f), u2 = (h2 >> 8) * (1.0f / 16777216.0f);
                const float r = sqrtf(-2.0f * logf(u1));
                a[p][i] = (half_t)(r * cosf(6.2831853f * u2));
                b[p][i] = (half_t)(0.02f * r * sinf(6.2831853f * u2));
            }
        }
    }
    float s = 0.f;
    if constexpr (SMALL) {
        float4_t acc[32];
#pragma unroll
        for (int j = 0; j < 32; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[j][e] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < 32; ++j)
                // written as text so that every accumulator stays in place (the builtin form made the register
                // allocator copy half of them through a scratch tuple around each MFMA)
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[j]) : "v"(a[j & 3]), "v"(b[(j >> 2) & 3]));
        }
#pragma unroll
        for (int j = 0; j < 32; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) s += acc[j][e];
    } else {
        float16_t acc[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < 16; ++j)
                acc[j & 7] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j & 3], b[(j >> 2) & 3], acc[j & 7], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) s += acc[j][e];
    }
    if (s == 123.456f) sink[0] = s; // keeps the loop alive
}

extern "C" {

// Runs the probe for about `ms_target` milliseconds on the default stream and returns the sustained rate.
// kind: 0 constant operands, 1 random operands shaped like the prompt pass's (N(0,1) x N(0,0.02)), both with
// v_mfma_f32_32x32x16_f16; 2 and 3: the same with v_mfma_f32_16x16x32_f16.  Returns 0, or the hipError_t of the
// call that failed (1 for bad arguments).  Built into its own shared object (libllmcu_probe.so) that only
// `bench.py --ceiling` loads; the token-loop library does not carry it.
int mfma_probe(int kind, float ms_target, double *tflops, float *ms_out) {
    if (!tflops || kind < 0 || kind > 3 || !(ms_target > 0.f)) return 1;
    int dev = 0, cus = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err == hipSuccess) err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (err != hipSuccess) return (int)err;
    float *sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    const int grid = cus * 2; // 8 wavefronts per CU, two per SIMD
    auto run = [&](int iters, float *ms) -> hipError_t {
        hipError_t e = hipEventRecord(e0, nullptr);
        if (e != hipSuccess) return e;
        if (kind & 2) mfma_probe_kernel<true><<<dim3(grid), dim3(256), 0, nullptr>>>(sink, iters, kind);
        else mfma_probe_kernel<false><<<dim3(grid), dim3(256), 0, nullptr>>>(sink, iters, kind);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        if ((e = hipEventRecord(e1, nullptr)) != hipSuccess) return e;
        if ((e = hipEventSynchronize(e1)) != hipSuccess) return e;
        return hipEventElapsedTime(ms, e0, e1);
    };
    float ms = 0.f;
    int iters = 10000;
    err = hipMalloc((void **)&sink, 4);
    if (err == hipSuccess) err = hipEventCreate(&e0);
    if (err == hipSuccess) err = hipEventCreate(&e1);
    if (err == hipSuccess) err = run(iters, &ms); // calibration (and warm-up)
    if (err == hipSuccess) {
        double want = (double)iters * ms_target / (ms > 0.01f ? ms : 0.01f);
        if (want > 2.0e8) want = 2.0e8;
        iters = want < 1000 ? 1000 : (int)want;
        err = run(iters, &ms);
    }
    if (err == hipSuccess) {
        const double flops = (double)grid * 4 /*wavefronts*/ * iters * 16.0 * (2.0 * 32 * 32 * 16);
        *tflops = flops / (ms * 1e-3) / 1e12;
        if (ms_out) *ms_out = ms;
    }
    // every path releases what it took
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (sink) (void)hipFree(sink);
    return (int)err;
}

} // extern "C"
