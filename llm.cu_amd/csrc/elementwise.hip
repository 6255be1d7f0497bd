// HBM-bound elementwise / row-reduction kernels: BF16->FP16 conversion,
// embedding gather, RMSNorm, residual add, RoPE (+ KV-cache append).
// Everything moves 16 bytes per lane per access where alignment allows.
#include <cmath>

#include "common.hpp"
#include "rms_device.hpp"

// ---------------------------------------------------------------------------
// BF16 -> FP16.  fp32 = bits << 16 is exact; v_cvt_f16_f32 rounds to nearest
// even; NaN is canonicalised to 0x7FFF (what __float2half_rn gives).
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint16_t cvt_bf16_fp16(uint16_t b) {
    float f = __uint_as_float((uint32_t)b << 16);
    half_t h = (half_t)f;
    uint16_t r = __builtin_bit_cast(uint16_t, h);
    return (f != f) ? (uint16_t)0x7fffu : r;
}

__global__ __launch_bounds__(256) void bf16_to_fp16_kernel(const uint16_t *__restrict__ src,
                                                           uint16_t *__restrict__ dst, size_t n_vec,
                                                           size_t n) {
    // each thread converts 8 elements per iteration (one 16-byte load, one 16-byte store)
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n_vec; i += stride) {
        uint4_t v = reinterpret_cast<const uint4_t *>(src)[i];
        uint4_t o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t w = v[j];
            uint32_t lo = cvt_bf16_fp16((uint16_t)(w & 0xffffu));
            uint32_t hi = cvt_bf16_fp16((uint16_t)(w >> 16));
            o[j] = lo | (hi << 16);
        }
        reinterpret_cast<uint4_t *>(dst)[i] = o;
    }
    // tail (< 8 elements) by the first threads of block 0
    if (blockIdx.x == 0) {
        size_t t = n_vec * 8 + threadIdx.x;
        if (t < n) dst[t] = cvt_bf16_fp16(src[t]);
    }
}

__global__ __launch_bounds__(256) void bf16_to_fp16_scalar_kernel(const uint16_t *__restrict__ src,
                                                                  uint16_t *__restrict__ dst, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = cvt_bf16_fp16(src[i]);
}

// ---------------------------------------------------------------------------
// Embedding gather: one block per token, 16-byte copies.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void embed_kernel(const half_t *__restrict__ table,
                                                    const int32_t *__restrict__ ids,
                                                    const int32_t *__restrict__ ids_offset,
                                                    half_t *__restrict__ out, int d, int vocab) {
    const int t = blockIdx.x;
    const int id = ids[t + (ids_offset ? *ids_offset : 0)];
    const bool ok = id >= 0 && id < vocab;
    const half_t *row = table + (size_t)(ok ? id : 0) * d;
    half_t *o = out + (size_t)t * d;
    for (int c = threadIdx.x * 8; c < d; c += blockDim.x * 8) {
        half8_t v = load8(row + c);
        if (!ok) {
            const half_t nanv = __builtin_bit_cast(half_t, (uint16_t)0x7fffu);
            v = half8_t{nanv, nanv, nanv, nanv, nanv, nanv, nanv, nanv};
        }
        store8(o + c, v);
    }
}

// ---------------------------------------------------------------------------
// Residual add: x = fp16(float(x) + float(res)).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void add_residual_kernel(half_t *__restrict__ x,
                                                           const half_t *__restrict__ res, size_t n_vec,
                                                           size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n_vec; i += stride) {
        half8_t a = load8(x + i * 8), b = load8(res + i * 8);
        half8_t o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (half_t)((float)a[j] + (float)b[j]);
        store8(x + i * 8, o);
    }
    if (blockIdx.x == 0) {
        size_t t = n_vec * 8 + threadIdx.x;
        if (t < n) x[t] = (half_t)((float)x[t] + (float)res[t]);
    }
}

// ---------------------------------------------------------------------------
// RMSNorm: one block per row (see rms_device.hpp for the summation order).
// ---------------------------------------------------------------------------
template <int THREADS>
__global__ __launch_bounds__(THREADS) void rmsnorm_kernel(const half_t *x, // may alias y
                                                          const half_t *__restrict__ gain,
                                                          half_t *y, int d, double eps) {
    __shared__ float red[THREADS + 1];
    const size_t row = blockIdx.x;
    rms_normalise_row<THREADS>(x + row * d, gain, y + row * d, d, eps, red);
}

// ---------------------------------------------------------------------------
// RoPE on adjacent pairs, angles from a host-built (cos, sin) table.
// Each thread rotates 4 pairs (8 halves, one 16-byte access).
// e' = c*e - s*o, o' = s*e + c*o with unfused multiplies (this file is
// compiled with -ffp-contract=off).
// ---------------------------------------------------------------------------
__device__ __forceinline__ half8_t rotate8(half8_t v, const float *__restrict__ cs) { return rope_rotate8(v, cs); }

__global__ __launch_bounds__(256) void rope_kernel(half_t *__restrict__ buf, int n_heads, int head_dim,
                                                   int row_stride, int pos0,
                                                   const int32_t *__restrict__ pos_dev,
                                                   const float *__restrict__ table, int max_pos) {
    const int t = blockIdx.y;
    const int width = n_heads * head_dim;
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (c >= width) return;
    int pos = pos0 + t + (pos_dev ? *pos_dev : 0);
    if (pos >= max_pos) pos = max_pos - 1; // host checks the range; never index past the table
    const int half = head_dim / 2;
    const int i0 = (c % head_dim) / 2; // first pair index inside the head
    const float *cs = table + ((size_t)pos * half + i0) * 2;
    half_t *p = buf + (size_t)t * row_stride + c;
    store8(p, rotate8(load8(p), cs));
}

// Fused: rotate Q in place, rotate K into the cache, copy V into the
// (position-contiguous) V cache.  qkv row: [Hq*hd | Hkv*hd | Hkv*hd].
// K cache: [Hkv][max_pos][hd]; V cache: [Hkv][hd][max_pos].
__global__ __launch_bounds__(256) void rope_kv_append_kernel(half_t *__restrict__ qkv,
                                                             half_t *__restrict__ kc,
                                                             half_t *__restrict__ vc, int n_heads,
                                                             int n_kv_heads, int head_dim, int pos0,
                                                             const int32_t *__restrict__ pos_dev,
                                                             const float *__restrict__ table,
                                                             int max_pos) {
    const int t = blockIdx.y;
    const int qd = n_heads * head_dim, kvd = n_kv_heads * head_dim;
    const int width = qd + 2 * kvd;
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (c >= width) return;
    int pos = pos0 + t + (pos_dev ? *pos_dev : 0);
    if (pos >= max_pos) pos = max_pos - 1;
    const int half = head_dim / 2;
    half_t *p = qkv + (size_t)t * width + c;
    half8_t v = load8(p);
    if (c < qd + kvd) {
        const int i0 = (c % head_dim) / 2;
        const float *cs = table + ((size_t)pos * half + i0) * 2;
        half8_t r = rotate8(v, cs);
        if (c < qd) {
            store8(p, r);
        } else {
            const int ck = c - qd;
            const int kvh = ck / head_dim, dd = ck % head_dim;
            store8(kc + ((size_t)kvh * max_pos + pos) * head_dim + dd, r);
        }
    } else {
        const int cv = c - qd - kvd;
        const int kvh = cv / head_dim, dd = cv % head_dim;
        half_t *dst = vc + ((size_t)kvh * head_dim + dd) * max_pos + pos;
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[(size_t)j * max_pos] = v[j];
    }
}

// V part for many rows at once: transposes a [64 positions x 64 dims] tile
// through LDS so that both the read (dims contiguous) and the write
// (positions contiguous) are coalesced.
__global__ __launch_bounds__(256) void v_append_transpose_kernel(const half_t *__restrict__ qkv,
                                                                 half_t *__restrict__ vc, int T,
                                                                 int n_heads, int n_kv_heads,
                                                                 int head_dim, int pos0, int max_pos) {
    __shared__ half_t tile[64][64 + 2];
    const int qd = n_heads * head_dim, kvd = n_kv_heads * head_dim;
    const int width = qd + 2 * kvd;
    const int t0 = blockIdx.x * 64;  // token tile
    const int c0 = blockIdx.y * 64;  // column tile inside the V part (kvd columns)
    // read: 64 rows x 64 cols, 8 halves per thread-load -> 512 loads, 2 per thread
    for (int i = threadIdx.x; i < 512; i += 256) {
        int r = i / 8, cc = (i % 8) * 8;
        half8_t v = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        if (t0 + r < T && c0 + cc < kvd) v = load8(qkv + (size_t)(t0 + r) * width + qd + kvd + c0 + cc);
#pragma unroll
        for (int j = 0; j < 8; ++j) tile[r][cc + j] = v[j];
    }
    __syncthreads();
    // write: for column c (a (kvh, dd) pair) positions t0..t0+63 are contiguous in the cache.  With whole groups of
    // eight positions on 16-byte boundaries a thread stores eight of them at once.
    if (((pos0 + t0) & 7) == 0 && (max_pos & 7) == 0 && ((uintptr_t)vc & 15u) == 0 && t0 + 64 <= T && c0 + 64 <= kvd) {
        for (int i = threadIdx.x; i < 512; i += 256) {
            const int cc = i / 8, r8 = (i % 8) * 8;
            half8_t v;
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = tile[r8 + j][cc];
            const int col = c0 + cc;
            const int kvh = col / head_dim, dd = col % head_dim;
            store8(vc + ((size_t)kvh * head_dim + dd) * max_pos + pos0 + t0 + r8, v);
        }
        return;
    }
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        int cc = i / 64, r = i % 64;
        int col = c0 + cc;
        if (t0 + r < T && col < kvd) {
            int kvh = col / head_dim, dd = col % head_dim;
            vc[((size_t)kvh * head_dim + dd) * max_pos + pos0 + t0 + r] = tile[r][cc];
        }
    }
}

// Q and K parts only (used with v_append_transpose_kernel when T is large).
__global__ __launch_bounds__(256) void rope_qk_append_kernel(half_t *__restrict__ qkv,
                                                             half_t *__restrict__ kc, int n_heads,
                                                             int n_kv_heads, int head_dim, int pos0,
                                                             const float *__restrict__ table,
                                                             int max_pos, int c_begin) {
    // c_begin: 0, or the width of Q when the queries stay as they are (the attention kernel rotates them itself)
    const int t = blockIdx.y;
    const int qd = n_heads * head_dim, kvd = n_kv_heads * head_dim;
    const int width = qd + 2 * kvd;
    const int c = c_begin + (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (c >= qd + kvd) return;
    int pos = pos0 + t;
    if (pos >= max_pos) pos = max_pos - 1;
    const int half = head_dim / 2;
    half_t *p = qkv + (size_t)t * width + c;
    const int i0 = (c % head_dim) / 2;
    const float *cs = table + ((size_t)pos * half + i0) * 2;
    half8_t r = rotate8(load8(p), cs);
    if (c < qd) {
        store8(p, r);
    } else {
        const int ck = c - qd;
        const int kvh = ck / head_dim, dd = ck % head_dim;
        store8(kc + ((size_t)kvh * max_pos + pos) * head_dim + dd, r);
    }
}

// ---------------------------------------------------------------------------
extern "C" {

int llm_bf16_to_fp16(const uint16_t *src, uint16_t *dst, size_t n, llm_stream_t stream) {
    LLM_REQUIRE(src && dst, "llm_bf16_to_fp16: null pointer");
    if (n == 0) return LLM_OK;
    hipStream_t s = (hipStream_t)stream;
    if (aligned16(src) && aligned16(dst)) {
        size_t n_vec = n / 8;
        size_t blocks = (n_vec + 255) / 256;
        if (blocks == 0) blocks = 1;
        if (blocks > 256 * 64) blocks = 256 * 64; // grid-stride beyond 16 blocks per CU
        bf16_to_fp16_kernel<<<dim3((unsigned)blocks), dim3(256), 0, s>>>(src, dst, n_vec, n);
        LLM_LAUNCH_CHECK("bf16_to_fp16_kernel");
    } else {
        size_t blocks = (n + 255) / 256;
        if (blocks > 256 * 64) blocks = 256 * 64;
        bf16_to_fp16_scalar_kernel<<<dim3((unsigned)blocks), dim3(256), 0, s>>>(src, dst, n);
        LLM_LAUNCH_CHECK("bf16_to_fp16_scalar_kernel");
    }
    return LLM_OK;
}

int llm_embed_gather(const uint16_t *table, const int32_t *ids, const int32_t *ids_offset, uint16_t *out, int T,
                     int d, int vocab, llm_stream_t stream) {
    LLM_REQUIRE(table && ids && out, "llm_embed_gather: null pointer");
    LLM_REQUIRE(T >= 0 && d > 0 && d % 8 == 0 && vocab > 0, "llm_embed_gather: T=%d d=%d vocab=%d", T, d, vocab);
    LLM_REQUIRE(aligned16(table) && aligned16(out), "llm_embed_gather: pointers must be 16-byte aligned");
    if (T == 0) return LLM_OK;
    embed_kernel<<<dim3(T), dim3(256), 0, (hipStream_t)stream>>>((const half_t *)table, ids, ids_offset,
                                                                 (half_t *)out, d, vocab);
    LLM_LAUNCH_CHECK("embed_kernel");
    return LLM_OK;
}

int llm_add_residual(uint16_t *x, const uint16_t *res, size_t n, llm_stream_t stream) {
    LLM_REQUIRE(x && res, "llm_add_residual: null pointer");
    LLM_REQUIRE(aligned16(x) && aligned16(res), "llm_add_residual: pointers must be 16-byte aligned");
    if (n == 0) return LLM_OK;
    size_t n_vec = n / 8;
    size_t blocks = (n_vec + 255) / 256;
    if (blocks == 0) blocks = 1;
    if (blocks > 256 * 64) blocks = 256 * 64;
    add_residual_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
        (half_t *)x, (const half_t *)res, n_vec, n);
    LLM_LAUNCH_CHECK("add_residual_kernel");
    return LLM_OK;
}

int llm_rmsnorm(const uint16_t *x, const uint16_t *gain, uint16_t *y, int T, int d, double eps,
                llm_stream_t stream) {
    LLM_REQUIRE(x && gain && y, "llm_rmsnorm: null pointer");
    LLM_REQUIRE(T >= 0 && rms_shape_ok(d), "llm_rmsnorm: d=%d (need d/4 a power of two in [64, 4096])", d);
    LLM_REQUIRE(((uintptr_t)x & 7u) == 0 && ((uintptr_t)y & 7u) == 0 && ((uintptr_t)gain & 7u) == 0,
                "llm_rmsnorm: pointers must be 8-byte aligned");
    if (T == 0) return LLM_OK;
    hipStream_t s = (hipStream_t)stream;
    const int n = d / 4;
    constexpr int RMS_ROW_THREADS = 128;
    if (n >= 256 && n <= RMS_ROW_THREADS * RMS_MAX_R) {
        rmsnorm_kernel<RMS_ROW_THREADS><<<dim3(T), dim3(RMS_ROW_THREADS), 0, s>>>((const half_t *)x, (const half_t *)gain, (half_t *)y, d, eps);
    } else if (n >= 256) {
        rmsnorm_kernel<256><<<dim3(T), dim3(256), 0, s>>>((const half_t *)x, (const half_t *)gain, (half_t *)y, d, eps);
    } else if (n == 128) {
        rmsnorm_kernel<128><<<dim3(T), dim3(128), 0, s>>>((const half_t *)x, (const half_t *)gain, (half_t *)y, d, eps);
    } else {
        rmsnorm_kernel<64><<<dim3(T), dim3(64), 0, s>>>((const half_t *)x, (const half_t *)gain, (half_t *)y, d, eps);
    }
    LLM_LAUNCH_CHECK("rmsnorm_kernel");
    return LLM_OK;
}

int llm_rope_table_host(float *table, int max_pos, int head_dim, float theta) {
    LLM_REQUIRE(table && max_pos > 0 && head_dim > 0 && head_dim % 2 == 0, "llm_rope_table_host: bad argument");
    const int half = head_dim / 2;
    for (int pos = 0; pos < max_pos; ++pos)
        for (int i = 0; i < half; ++i) {
            float freq = 1.0f / powf(theta, 2.0f * (float)i / (float)head_dim);
            float angle = (float)pos * freq;
            table[((size_t)pos * half + i) * 2] = cosf(angle);
            table[((size_t)pos * half + i) * 2 + 1] = sinf(angle);
        }
    return LLM_OK;
}

int llm_rope(uint16_t *buf, int T, int n_heads, int head_dim, int row_stride, int pos0, const int32_t *pos_dev,
             const float *table, int max_pos, llm_stream_t stream) {
    LLM_REQUIRE(buf && table, "llm_rope: null pointer");
    LLM_REQUIRE(T >= 0 && n_heads > 0 && head_dim >= 8 && head_dim % 8 == 0, "llm_rope: bad shape");
    LLM_REQUIRE(row_stride >= n_heads * head_dim && row_stride % 8 == 0, "llm_rope: row_stride=%d", row_stride);
    LLM_REQUIRE(pos0 >= 0 && pos0 + T <= max_pos, "llm_rope: positions %d..%d exceed max_pos %d", pos0, pos0 + T, max_pos);
    LLM_REQUIRE(aligned16(buf), "llm_rope: buf must be 16-byte aligned");
    if (T == 0) return LLM_OK;
    const int width = n_heads * head_dim;
    dim3 grid((width / 8 + 255) / 256, T);
    rope_kernel<<<grid, dim3(256), 0, (hipStream_t)stream>>>((half_t *)buf, n_heads, head_dim, row_stride, pos0,
                                                             pos_dev, table, max_pos);
    LLM_LAUNCH_CHECK("rope_kernel");
    return LLM_OK;
}

static int rope_kv_append(uint16_t *qkv, uint16_t *kc, uint16_t *vc, int T, int n_heads, int n_kv_heads, int head_dim,
                          int pos0, const int32_t *pos_dev, const float *table, int max_pos, bool keep_q,
                          llm_stream_t stream) {
    LLM_REQUIRE(qkv && kc && vc && table, "llm_rope_kv_append: null pointer");
    LLM_REQUIRE(T >= 0 && n_heads > 0 && n_kv_heads > 0 && head_dim >= 8 && head_dim % 8 == 0,
                "llm_rope_kv_append: bad shape");
    LLM_REQUIRE(pos0 >= 0 && pos0 + T <= max_pos, "llm_rope_kv_append: positions %d..%d exceed max_pos %d", pos0,
                pos0 + T, max_pos);
    LLM_REQUIRE(aligned16(qkv) && aligned16(kc), "llm_rope_kv_append: pointers must be 16-byte aligned");
    if (T == 0) return LLM_OK;
    hipStream_t s = (hipStream_t)stream;
    const int qd = n_heads * head_dim, kvd = n_kv_heads * head_dim;
    LLM_REQUIRE(!keep_q || (T >= 16 && !pos_dev), "llm_rope_k_append: at least 16 rows at host-known positions");
    if (T < 16 || pos_dev) {
        dim3 grid(((qd + 2 * kvd) / 8 + 255) / 256, T);
        rope_kv_append_kernel<<<grid, dim3(256), 0, s>>>((half_t *)qkv, (half_t *)kc, (half_t *)vc, n_heads,
                                                         n_kv_heads, head_dim, pos0, pos_dev, table, max_pos);
        LLM_LAUNCH_CHECK("rope_kv_append_kernel");
    } else {
        const int c_begin = keep_q ? qd : 0;
        dim3 grid(((qd + kvd - c_begin) / 8 + 255) / 256, T);
        rope_qk_append_kernel<<<grid, dim3(256), 0, s>>>((half_t *)qkv, (half_t *)kc, n_heads, n_kv_heads, head_dim,
                                                         pos0, table, max_pos, c_begin);
        LLM_LAUNCH_CHECK("rope_qk_append_kernel");
        dim3 gv((T + 63) / 64, (kvd + 63) / 64);
        v_append_transpose_kernel<<<gv, dim3(256), 0, s>>>((const half_t *)qkv, (half_t *)vc, T, n_heads, n_kv_heads,
                                                           head_dim, pos0, max_pos);
        LLM_LAUNCH_CHECK("v_append_transpose_kernel");
    }
    return LLM_OK;
}

int llm_rope_kv_append(uint16_t *qkv, uint16_t *kc, uint16_t *vc, int T, int n_heads, int n_kv_heads, int head_dim,
                       int pos0, const int32_t *pos_dev, const float *table, int max_pos, llm_stream_t stream) {
    return rope_kv_append(qkv, kc, vc, T, n_heads, n_kv_heads, head_dim, pos0, pos_dev, table, max_pos, false, stream);
}

int llm_rope_k_append(uint16_t *qkv, uint16_t *kc, uint16_t *vc, int T, int n_heads, int n_kv_heads, int head_dim,
                      int pos0, const float *table, int max_pos, llm_stream_t stream) {
    return rope_kv_append(qkv, kc, vc, T, n_heads, n_kv_heads, head_dim, pos0, nullptr, table, max_pos, true, stream);
}

} // extern "C"
