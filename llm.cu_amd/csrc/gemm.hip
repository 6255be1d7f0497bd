// Projections for more than one token: out = x . w^T with fp32 accumulation
// on the MFMA units.  w is [N, K] row-major and x is [T, K] row-major, so both
// MFMA operands are K-contiguous and every lane's fragment is one 16-byte load.
//
//  * skinny (2 <= T <= 16): one workgroup per 16 weight rows, its 8 wavefronts
//    split K, v_mfma_f32_16x16x32_f16 with the token rows as the M side.
//    HBM-bound: weights are read once, straight from global memory.
//  * tiled GEMM (T > 16): BM x BN macro-tiles staged through LDS (double
//    buffered, padded rows), v_mfma_f32_32x32x16_f16, wave tiles up to 128x128.
//
// MFMA operand layouts used below (wave64):
//   16x16x32: A lane l -> row l%16, k = 8*(l/16)..+7;  B lane l -> col l%16, same k;
//             D lane l -> col l%16, rows 4*(l/16)+i, i<4.
//   32x32x16: A lane l -> row l%32, k = 8*(l/32)..+7;  B lane l -> col l%32, same k;
//             D lane l -> col l%32, rows 8*(i/4) + 4*(l/32) + i%4, i<16.
#include <cmath>
#include <mutex>
#include <type_traits>
#include <vector>

#include "common.hpp"

int gemv_launch(const half_t *x, const half_t *gain, double eps, const half_t *w, const half_t *res, half_t *out,
                int N, int K, hipStream_t s);
int gemv_swiglu_launch(const half_t *x, const half_t *gain, double eps, const half_t *wg, const half_t *wu,
                       half_t *out, int N, int K, hipStream_t s);
int gemv_embed_launch(const half_t *table, const int32_t *ids, const int32_t *ids_offset, int vocab, half_t *x_copy,
                      const half_t *gain, double eps, const half_t *w, half_t *out, int N, int K, hipStream_t s);


// address-space cast for the LDS side of the loads that go from global memory straight into LDS
#define DMA_LP(p) ((__attribute__((address_space(3))) void *)(p))

// ---------------------------------------------------------------------------
// skinny
// ---------------------------------------------------------------------------
#define SK_WAVES 8

template <bool SWIGLU>
__global__ __launch_bounds__(SK_WAVES * 64) void skinny_kernel(const half_t *__restrict__ x, int ldx,
                                                               const half_t *__restrict__ w,
                                                               const half_t *__restrict__ w2,
                                                               const half_t *res, int ldr, // may alias out
                                                               half_t *out, int ldo, int T,
                                                               int N, int K) {
    __shared__ float red[SWIGLU ? 2 : 1][SK_WAVES][64][4];
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int r = lane % 16, g = lane / 16;
    const int n0 = blockIdx.x * 16;
    const int nrow = n0 + r < N ? n0 + r : N - 1;
    const int mrow = r < T ? r : T - 1;
    const int kslice = K / SK_WAVES; // multiple of 32
    const int kbeg = wave * kslice;
    const half_t *xp = x + (size_t)mrow * ldx + kbeg + 8 * g;
    const half_t *wp = w + (size_t)nrow * K + kbeg + 8 * g;
    const half_t *wp2 = SWIGLU ? w2 + (size_t)nrow * K + kbeg + 8 * g : nullptr;
    float4_t acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
    // Weights are read once (non-temporal), U k-steps per round; the loads of round i+1 are issued
    // before the MFMAs of round i (two register sets), so a wave always has a round in flight.
    constexpr int U = 4;
    half8_t a[2][U], b[2][U], b2[2][U];
    const int rounds = kslice / (32 * U);
    auto fetch = [&](int set, int k) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            b[set][u] = load8_nt(wp + k + 32 * u);
            if (SWIGLU) b2[set][u] = load8_nt(wp2 + k + 32 * u);
            a[set][u] = load8(xp + k + 32 * u);
        }
    };
    auto mma = [&](int set) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[set][u], b[set][u], acc, 0, 0, 0);
            if (SWIGLU) acc2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[set][u], b2[set][u], acc2, 0, 0, 0);
        }
    };
    if (rounds > 0) fetch(0, 0);
    int rd = 0;
    for (; rd + 2 <= rounds; rd += 2) { // unrolled by two so that the register-set index is a constant
        fetch(1, (rd + 1) * 32 * U);
        mma(0);
        if (rd + 2 < rounds) fetch(0, (rd + 2) * 32 * U);
        mma(1);
    }
    if (rd < rounds) mma(0);
    for (int k = rounds * 32 * U; k < kslice; k += 32) {
        half8_t av = load8(xp + k), bv = load8(wp + k);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, acc, 0, 0, 0);
        if (SWIGLU) acc2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, load8(wp2 + k), acc2, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        red[0][wave][lane][i] = acc[i];
        if (SWIGLU) red[SWIGLU ? 1 : 0][wave][lane][i] = acc2[i];
    }
    __syncthreads();
    if (wave == 0) {
        const int n = n0 + lane % 16;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = 4 * (lane / 16) + i;
            float s = 0.f, s2 = 0.f;
#pragma unroll
            for (int wv = 0; wv < SK_WAVES; ++wv) {
                s += red[0][wv][lane][i];
                if (SWIGLU) s2 += red[SWIGLU ? 1 : 0][wv][lane][i];
            }
            if (m < T && n < N) {
                if (SWIGLU) {
                    out[(size_t)m * ldo + n] = swiglu_to_half(s, s2);
                } else {
                    out[(size_t)m * ldo + n] = finish(s, res ? res + (size_t)m * ldr + n : nullptr);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// skinny, weights through LDS
// ---------------------------------------------------------------------------
// The kernel above reads, per load instruction, 64 bytes from each of 16 weight rows.  Here every wave
// instruction moves 512 contiguous bytes of two rows straight into the wave's own LDS tile
// (buffer_load ... lds), i.e. the DRAM pattern of the GEMV, and the MFMA fragments are read back from LDS.
// Same work split: workgroup = 16 output columns, WAVES wavefronts each own a k-slice and process it in
// chunks of 256; D + 1 chunks per wave are in LDS, one being consumed while the next ones land (no
// workgroup barrier: the tiles are private to the wave).  Measured at the 8B shapes, a ring of two tiles
// with four waves is as fast as or faster than deeper rings or more waves.  Lane l of an instruction fetches 16-byte chunk
// (l%32) ^ (row&15) of its row so that the 16 rows a fragment read touches per cycle sit in 16
// different bank groups.
#define SKD_CHUNK 256

template <int N> __device__ __forceinline__ void skd_wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// D = chunks in flight ahead of the one being consumed (LDS ring of D + 1 tiles per wave). N % 16 == 0.
// XLDS: the x chunk travels like a weight tile (row-contiguous loads into LDS, fragments read back from
// there) instead of straight into registers, where one load instruction touches 16 rows of 64 bytes.
template <bool SWIGLU, int WAVES, int D, bool XLDS>
__global__ __launch_bounds__(WAVES * 64, 1) void skinny_dma_kernel(const half_t *__restrict__ x, int ldx,
                                                                   const half_t *__restrict__ w,
                                                                   const half_t *__restrict__ w2, const half_t *res,
                                                                   int ldr, half_t *out, int ldo, int T, int N, int K) {
    constexpr int NW = SWIGLU ? 2 : 1;
    constexpr int NS = D + 1;                         // ring slots = register sets
    constexpr int TILE = 16 * SKD_CHUNK;              // halves per weight tile (8 KB)
    constexpr int VM = 8 * NW + 8;                    // load instructions a chunk issues (weights + x)
    static_assert(D >= 1 && D <= 3 && D * VM <= 63, "vmcnt counts at most 63 outstanding loads");
    constexpr int SLOT = (NW + (XLDS ? 1 : 0)) * TILE; // halves per ring slot
    extern __shared__ __attribute__((aligned(16))) half_t sk_lds[]; // [WAVES][NS][SLOT]
    __shared__ float red[2][NW][WAVES][64][4];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
    const int r = lane % 16, g = lane / 16;
    const int mrow = r < T ? r : T - 1;
    const int kslice = K / WAVES; // multiple of SKD_CHUNK
    const int kbeg = wave * kslice;
    const int nchunks = kslice / SKD_CHUNK;
    half_t *mine = sk_lds + (size_t)wave * NS * SLOT;
    // The workgroup walks over column tiles blockIdx.x, blockIdx.x + gridDim.x, ...; its waves see one
    // flat sequence of (tile, chunk) items, so the first chunks of the next tile are already on their
    // way while the last chunk of the current one is consumed and reduced.
    const int n_tiles = N / 16;

    // element offset of this lane's 16 bytes inside a tile, per load instruction (two rows each)
    uint32_t lane_off[8], lane_off_x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int row = 2 * j + lane / 32;
        const uint32_t swz = (uint32_t)(((lane % 32) ^ (row & 15)) * 8);
        lane_off[j] = (uint32_t)row * (uint32_t)K + swz;
        if (XLDS) lane_off_x[j] = (uint32_t)(row < T ? row : T - 1) * (uint32_t)ldx + swz;
    }
    const half_t *xrow = x + (size_t)mrow * ldx + kbeg + 8 * g;
    half8_t a[XLDS ? 1 : NS][8];
    // Loads are issued at every ring step, also past the last item: there all lanes fetch the first 16
    // bytes of the weights (one cache line, never consumed). The number of loads in flight is then the
    // same at every step, so one constant vmcnt marks the arrival of the item about to be consumed.
    // The weights go to LDS through buffer loads: with the flat-encoded LDS loads in flight the compiler
    // turns every wait for the x registers into a wait for all loads, which empties the ring.
    const int w_bytes = N * K * (int)sizeof(half_t); // < 2^31, checked by the launcher
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void *)w, 0, w_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_w2 = __builtin_amdgcn_make_buffer_rsrc((void *)(SWIGLU ? w2 : w), 0, w_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_x =
        __builtin_amdgcn_make_buffer_rsrc((void *)x, 0, ((T - 1) * ldx + K) * (int)sizeof(half_t), 0x00020000);
    int c_tile = blockIdx.x, c_chunk = 0; // issue cursor
    auto issue = [&](int slot) {
        const bool live = c_tile < n_tiles;
        const uint32_t keep = live ? 0xffffffffu : 0u;
        const uint32_t base = live ? ((uint32_t)c_tile * 16u * (uint32_t)K + kbeg + c_chunk * SKD_CHUNK) * 2u : 0u;
        half_t *st = mine + (size_t)slot * SLOT;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t off = (lane_off[j] & keep) * 2u;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, DMA_LP(st + 2 * j * SKD_CHUNK), 16, off, base, 0, 0);
            if (SWIGLU)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w2, DMA_LP(st + TILE + 2 * j * SKD_CHUNK), 16, off, base, 0, 0);
        }
        // x is always read at the cursor's chunk (valid also past the last item); the empty asm hides the
        // offset from the optimiser, which would otherwise replace a repeated load by a register copy
        // and change the number of loads in flight
        int xoff = c_chunk * SKD_CHUNK;
        if (XLDS) {
            const uint32_t xbase = (uint32_t)(kbeg + xoff) * 2u;
#pragma unroll
            for (int j = 0; j < 8; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, DMA_LP(st + NW * TILE + 2 * j * SKD_CHUNK), 16,
                                                         lane_off_x[j] * 2u, xbase, 0, 0);
        } else {
            asm volatile("" : "+s"(xoff));
            const half_t *xs = xrow + xoff;
#pragma unroll
            for (int u = 0; u < 8; ++u) a[slot][u] = load8(xs + 32 * u);
        }
        if (++c_chunk == nchunks) {
            c_chunk = 0;
            c_tile += gridDim.x;
        }
    };
    float4_t acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
    auto consume = [&](int slot) {
        const half_t *st = mine + (size_t)slot * SLOT + r * SKD_CHUNK;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int pch = (4 * u + g) ^ r; // r < 16
            const half8_t b = load8(st + pch * 8);
            const half8_t af = XLDS ? load8(st + NW * TILE + pch * 8) : a[XLDS ? 0 : slot][u];
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, b, acc, 0, 0, 0);
            if (SWIGLU) {
                const half8_t b2 = load8(st + TILE + pch * 8);
                acc2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, b2, acc2, 0, 0, 0);
            }
        }
    };
    // End of a tile: the k-slices of the waves are added in wave order by one wave, which then runs the
    // epilogue. The partial sums alternate between two buffers, so one barrier per tile is enough (a wave
    // reaches the buffer of tile t again only behind the barrier of tile t + 1), and the epilogue wave
    // rotates, so the wait for the residual values is not always the same wave's.
    int u_tile = blockIdx.x, u_chunk = 0, flip = 0, ep_wave = 0; // consume cursor
    auto flush = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            red[flip][0][wave][lane][i] = acc[i];
            if (SWIGLU) red[flip][NW - 1][wave][lane][i] = acc2[i];
            acc[i] = 0.f;
            acc2[i] = 0.f;
        }
        // workgroup barrier without a wait on the loads in flight
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (wave == ep_wave) {
            const int n = u_tile * 16 + lane % 16;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = 4 * (lane / 16) + i;
                float s = 0.f, s2 = 0.f;
#pragma unroll
                for (int wv = 0; wv < WAVES; ++wv) {
                    s += red[flip][0][wv][lane][i];
                    if (SWIGLU) s2 += red[flip][NW - 1][wv][lane][i];
                }
                if (m < T) {
                    if (SWIGLU) out[(size_t)m * ldo + n] = swiglu_to_half(s, s2);
                    else out[(size_t)m * ldo + n] = finish(s, res ? res + (size_t)m * ldr + n : nullptr);
                }
            }
        }
        flip ^= 1;
        ep_wave = ep_wave + 1 == WAVES ? 0 : ep_wave + 1;
    };
    // one step with compile-time ring slot SLOT: refill the slot freed by the previous step, wait for
    // this item's loads, consume
    auto step = [&](auto slot_tag) {
        constexpr int SLOT = decltype(slot_tag)::value;
        issue((SLOT + D) % NS);
        skd_wait_vm<D * VM>();
        if (u_tile < n_tiles) {
            consume(SLOT);
            // the reads of this slot must have returned before the next step refills it
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (++u_chunk == nchunks) {
                flush();
                u_chunk = 0;
                u_tile += gridDim.x;
            }
        }
    };
#pragma unroll
    for (int i = 0; i < D; ++i) issue(i);
    while (u_tile < n_tiles) {
        step(std::integral_constant<int, 0>{});
        if (NS > 1) step(std::integral_constant<int, 1 % NS>{});
        if (NS > 2) step(std::integral_constant<int, 2 % NS>{});
        if (NS > 3) step(std::integral_constant<int, 3 % NS>{});
    }
    skd_wait_vm<0>(); // the filler loads still write into this workgroup's LDS
}

// whole 16-column tiles, and byte offsets into the weights that fit the 32-bit buffer addressing
static bool skd_fits(int N, int K) { return N % 16 == 0 && (size_t)N * K * sizeof(half_t) < ((size_t)1 << 31); }

template <bool SWIGLU, int WAVES, int D, bool XLDS>
static int skinny_dma_launch(const half_t *x, int ldx, const half_t *w, const half_t *w2, const half_t *res, int ldr,
                             half_t *out, int ldo, int T, int N, int K, hipStream_t s) {
    const size_t smem = sizeof(half_t) * (size_t)WAVES * (D + 1) * ((SWIGLU ? 2 : 1) + (XLDS ? 1 : 0)) * 16 * SKD_CHUNK;
    static_assert(sizeof(half_t) * WAVES * (D + 1) * ((SWIGLU ? 2 : 1) + (XLDS ? 1 : 0)) * 16 * SKD_CHUNK <= 144 * 1024,
                  "ring does not fit beside the reduction buffers");
    auto kern = skinny_dma_kernel<SWIGLU, WAVES, D, XLDS>;
    static std::atomic<uint64_t> attr_done{0};
    int rc = llm_ensure_max_smem((const void *)kern, smem, attr_done);
    if (rc != LLM_OK) return rc;
    // the LDS tiles allow one workgroup per CU: as many workgroups as CUs, each walking over column tiles
    int cus = 0;
    rc = llm_cu_count_cached(&cus);
    if (rc != LLM_OK) return rc;
    const int tiles = (N + 15) / 16;
    kern<<<dim3(tiles < cus ? tiles : cus), dim3(WAVES * 64), smem, s>>>(x, ldx, w, w2, res, ldr, out, ldo, T, N, K);
    LLM_LAUNCH_CHECK("skinny_dma_kernel");
    return LLM_OK;
}

// ---------------------------------------------------------------------------
// tiled MFMA GEMM
// ---------------------------------------------------------------------------
#define GEMM_BK 64
#define GEMM_PAD 8
#define GEMM_LD (GEMM_BK + GEMM_PAD) // LDS row stride in halves: 144 B, so 8 rows hit 8 different 16-byte bank groups

enum { EPI_PLAIN = 0, EPI_SWIGLU = 1 };

// BM x BN macro-tile, WGM x WGN wavefronts, NB = number of weight matrices
// (2 for the fused gate/up pair: BN rows of each).
template <int BM, int BN, int WGM, int WGN, int NB>
__global__ __launch_bounds__(WGM *WGN * 64) void gemm_kernel(const half_t *__restrict__ x, int ldx,
                                                             const half_t *__restrict__ w,
                                                             const half_t *__restrict__ w2,
                                                             const half_t *res, int ldr, // may alias out
                                                             half_t *out, int ldo, int T,
                                                             int N, int K, int tiles_m, int tiles_n) {
    constexpr int THREADS = WGM * WGN * 64;
    constexpr int TM = BM / WGM, TN = BN / WGN; // wave tile
    constexpr int FM = TM / 32, FN = TN / 32;   // 32x32 fragments per wave
    constexpr int A_LOADS = BM * GEMM_BK / 8 / THREADS;
    constexpr int B_LOADS = BN * GEMM_BK / 8 / THREADS;
    static_assert(A_LOADS >= 1 && B_LOADS >= 1, "tile too small for the workgroup");
    static_assert(BM * GEMM_BK / 8 % THREADS == 0 && BN * GEMM_BK / 8 % THREADS == 0, "uneven staging");

    extern __shared__ __attribute__((aligned(16))) half_t lds[];
    half_t *As = lds;                                    // [2][BM][GEMM_LD]
    half_t *Bs = lds + 2 * BM * GEMM_LD;                 // [2][NB][BN][GEMM_LD]

    // XCD-aware tile order.  Consecutive workgroup ids land on different XCDs
    // (8 of them, each with its own L2), so each XCD first gets a contiguous
    // run of logical tiles; inside a run the tiles walk GROUP_M rows of M for
    // every N column, so the ~32 tiles an XCD works on at a time form a compact
    // 8 x 4 block that shares its A rows and B rows through that XCD's L2.
    const int nblk = tiles_m * tiles_n;
    int bid = blockIdx.x;
    {
        const int per = nblk / 8;
        if (per > 0 && bid < per * 8) bid = (bid % 8) * per + bid / 8;
    }
    constexpr int GROUP_M = 8;
    const int group = bid / (GROUP_M * tiles_n);
    const int first_m = group * GROUP_M;
    const int gsz = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
    const int tm = first_m + (bid % (GROUP_M * tiles_n)) % gsz;
    const int tn = (bid % (GROUP_M * tiles_n)) / gsz;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int wm = wave % WGM, wn = wave / WGM;

    // staging map: 8 threads cover one 64-half row
    const int srow = tid / 8, scol = (tid % 8) * 8;
    constexpr int ROWS_PER_PASS = THREADS / 8;

    const half_t *ag[A_LOADS];
    const half_t *bg[NB][B_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        int row = m0 + srow + i * ROWS_PER_PASS;
        row = row < T ? row : T - 1;
        ag[i] = x + (size_t)row * ldx + scol;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
        int row = n0 + srow + i * ROWS_PER_PASS;
        row = row < N ? row : N - 1;
        bg[0][i] = w + (size_t)row * K + scol;
        if (NB == 2) bg[NB - 1][i] = w2 + (size_t)row * K + scol;
    }

    float16_t acc[NB][FM][FN];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[b][i][j][e] = 0.f;

    // Global loads run DEPTH k-tiles ahead of the MFMAs through DEPTH register
    // sets: tile kt+DEPTH is requested at the top of iteration kt, and tile kt+1
    // (requested DEPTH iterations earlier) is written to the other LDS buffer at
    // the bottom, so a trip to HBM has DEPTH iterations of matrix work to hide
    // behind.  One wavefront per SIMD (4-wave tiles) has the registers for two.
    constexpr int DEPTH = (WGM * WGN <= 4) ? 2 : 1;
    half8_t ra[DEPTH][A_LOADS], rb[DEPTH][NB][B_LOADS];
    auto gload = [&](int set, int k0) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) ra[set][i] = load8(ag[i] + k0);
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int i = 0; i < B_LOADS; ++i) rb[set][b][i] = load8(bg[b][i] + k0);
    };
    auto sstore = [&](int set, int buf) {
        half_t *a = As + buf * BM * GEMM_LD;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) store8(a + (srow + i * ROWS_PER_PASS) * GEMM_LD + scol, ra[set][i]);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            half_t *bb = Bs + (buf * NB + b) * BN * GEMM_LD;
#pragma unroll
            for (int i = 0; i < B_LOADS; ++i) store8(bb + (srow + i * ROWS_PER_PASS) * GEMM_LD + scol, rb[set][b][i]);
        }
    };
    const int frow = lane % 32, fk = (lane / 32) * 8;
    // Fragments of k-step ks+1 are read from LDS while the MFMAs of k-step ks
    // run (two fragment register sets), so LDS latency sits behind matrix work.
    auto compute = [&](int buf) {
        const half_t *a = As + buf * BM * GEMM_LD + (wm * TM + frow) * GEMM_LD + fk;
        const half_t *bp[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) bp[b] = Bs + (buf * NB + b) * BN * GEMM_LD + (wn * TN + frow) * GEMM_LD + fk;
        half8_t af[2][FM], bf[2][NB][FN];
        auto lfrag = [&](int set, int ks) {
#pragma unroll
            for (int i = 0; i < FM; ++i) af[set][i] = load8(a + i * 32 * GEMM_LD + ks * 16);
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int j = 0; j < FN; ++j) bf[set][b][j] = load8(bp[b] + j * 32 * GEMM_LD + ks * 16);
        };
        lfrag(0, 0);
#pragma unroll
        for (int ks = 0; ks < GEMM_BK / 16; ++ks) {
            const int cur = ks & 1;
            if (ks + 1 < GEMM_BK / 16) lfrag(cur ^ 1, ks + 1);
            __builtin_amdgcn_sched_barrier(0); // keep the LDS reads ahead of this step's MFMAs
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j)
                        acc[b][i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[cur][i], bf[cur][b][j], acc[b][i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int nk = K / GEMM_BK;
    gload(0, 0);
    sstore(0, 0);
    if (DEPTH == 2 && nk > 1) gload(DEPTH - 1, GEMM_BK);
    __syncthreads();
    // unrolled by two so that register-set and LDS-buffer indices are constants:
    // iteration kt uses LDS buffer kt%2; with DEPTH 2, tile kt+1 sits in register set (kt+1)%2
    for (int kt = 0; kt < nk; kt += 2) {
        if (kt + DEPTH < nk) gload(0, (kt + DEPTH) * GEMM_BK);
        compute(0);
        if (kt + 1 < nk) sstore(DEPTH - 1, 1);
        __syncthreads();
        if (kt + 1 < nk) {
            if (kt + 1 + DEPTH < nk) gload(DEPTH - 1, (kt + 1 + DEPTH) * GEMM_BK);
            compute(1);
            if (kt + 2 < nk) sstore(0, 0);
            __syncthreads();
        }
    }

    // epilogue: D lane l -> col l%32, rows 8*(e/4) + 4*(l/32) + e%4
    const int ccol = lane % 32, crow0 = 4 * (lane / 32);
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int n = n0 + wn * TN + j * 32 + ccol;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * TM + i * 32 + 8 * (e / 4) + crow0 + (e % 4);
                if (m < T && n < N) {
                    if (NB == 2) {
                        out[(size_t)m * ldo + n] = swiglu_to_half(acc[0][i][j][e], acc[NB - 1][i][j][e]);
                    } else {
                        out[(size_t)m * ldo + n] = finish(acc[0][i][j][e], res ? res + (size_t)m * ldr + n : nullptr);
                    }
                }
            }
        }
}

template <int BM, int BN, int WGM, int WGN, int NB>
static int gemm_launch(const half_t *x, int ldx, const half_t *w, const half_t *w2, const half_t *res, int ldr,
                       half_t *out, int ldo, int T, int N, int K, hipStream_t s) {
    const int tiles_m = (T + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const size_t smem = sizeof(half_t) * (2 * (size_t)BM * GEMM_LD + 2 * (size_t)NB * BN * GEMM_LD);
    auto kern = gemm_kernel<BM, BN, WGM, WGN, NB>;
    static std::atomic<uint64_t> attr_done{0};
    if (smem > 48 * 1024) {
        int rc = llm_ensure_max_smem((const void *)kern, smem, attr_done);
        if (rc != LLM_OK) return rc;
    }
    kern<<<dim3(tiles_m * tiles_n), dim3(WGM * WGN * 64), smem, s>>>(x, ldx, w, w2, res, ldr, out, ldo, T, N, K,
                                                                     tiles_m, tiles_n);
    LLM_LAUNCH_CHECK("gemm_kernel");
    return LLM_OK;
}

// ---------------------------------------------------------------------------
// large-T MFMA GEMM: tiles go from global memory straight into LDS
// ---------------------------------------------------------------------------
// No register staging: every wavefront issues buffer loads with LDS destination (16 B per lane, 1 KB per
// instruction, landing contiguously in LDS), STAGES buffers deep, and waits with an explicit vmcnt so that loads
// stay in flight across workgroup barriers.  Because a wave instruction fills 16 consecutive 64-byte
// rows, the row padding of the kernel above is not available; instead lane l fetches global 16-byte
// chunk (l%4) ^ ((row>>2)&3) of its row, so that the 16 lanes an LDS read serves per cycle (16 rows,
// same logical chunk) fall into 16 different 16-byte bank groups.
#define DMA_BK 32

template <int N> __device__ __forceinline__ void dma_wait_barrier() {
    // vmcnt(N): all but the newest N of this wave's loads have landed; then the workgroup barrier.
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}
// the same with a run-time number of tiles (of LPT loads each, at most MAXT) allowed to stay in flight
template <int LPT, int MAXT> __device__ __forceinline__ void dma_wait_tiles(int tiles) {
    static_assert(MAXT * LPT <= 63, "vmcnt counts at most 63 outstanding loads");
    if (MAXT >= 7 && tiles >= 7) dma_wait_barrier<(MAXT >= 7 ? 7 : 0) * LPT>();
    else if (MAXT >= 6 && tiles >= 6) dma_wait_barrier<(MAXT >= 6 ? 6 : 0) * LPT>();
    else if (MAXT >= 5 && tiles >= 5) dma_wait_barrier<(MAXT >= 5 ? 5 : 0) * LPT>();
    else if (MAXT >= 4 && tiles >= 4) dma_wait_barrier<(MAXT >= 4 ? 4 : 0) * LPT>();
    else if (MAXT >= 3 && tiles >= 3) dma_wait_barrier<(MAXT >= 3 ? 3 : 0) * LPT>();
    else if (MAXT >= 2 && tiles >= 2) dma_wait_barrier<(MAXT >= 2 ? 2 : 0) * LPT>();
    else if (MAXT >= 1 && tiles >= 1) dma_wait_barrier<(MAXT >= 1 ? 1 : 0) * LPT>();
    else dma_wait_barrier<0>();
}

// (WGM*FM*32) x (WGN*128) macro-tile, WGM*WGN wavefronts each owning (FM*32) x 128 of it (NB = 2: 64 columns of
// gate and the same 64 of up), BK = 32, STAGES LDS buffers filled by direct global->LDS loads.
// Split-K (ws != nullptr): workgroup (tile, z) covers k in [z*kper, (z+1)*kper) and stores its fp32
// partial tile to ws[z][T][N]; splitk_reduce_kernel sums the slices in ascending z and finishes.
// Loads run STAGES-1 tiles ahead.  PREF must be false: the pipeline that reads the next tile's first fragments
// before the barrier is gemm_dma64_kernel's (the 256 x 256 tile of the long prompt passes).
template <int NB, int WGM, int WGN, int STAGES, bool PREF, int OCC, int FM = 2>
__global__ __launch_bounds__(WGM * WGN * 64, OCC) void gemm_dma_kernel(const half_t *__restrict__ x, int ldx,
                                                               const half_t *__restrict__ w, const half_t *__restrict__ w2,
                                                               const half_t *res, int ldr, half_t *out, int ldo, int T, int N, int K,
                                                               int tiles_m, int tiles_n, float *ws, int kper) {
    constexpr int NWAVES = WGM * WGN;
    constexpr int WTM = FM * 32;                           // rows of a wave tile
    constexpr int BM = WGM * WTM, BROWS = WGN * 128;       // B rows in a stage (both matrices when NB = 2)
    constexpr int BN = BROWS / NB;             // output columns per tile
    constexpr int FN = 4 / NB;
    constexpr int STAGE_HALVES = (BM + BROWS) * DMA_BK;
    constexpr int LPT = (BM + BROWS) / 16 / NWAVES; // load instructions per wave per tile
    constexpr int AHEAD = PREF ? STAGES - 2 : STAGES - 1;
    extern __shared__ __attribute__((aligned(16))) half_t lds[];

    const int nblk = tiles_m * tiles_n;
    int bid = blockIdx.x;
    {
        const int per = nblk / 8;
        if (per > 0 && bid < per * 8) bid = (bid % 8) * per + bid / 8;
    }
    constexpr int GROUP_M = 8;
    const int group = bid / (GROUP_M * tiles_n);
    const int first_m = group * GROUP_M;
    const int gsz = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
    const int tm = first_m + (bid % (GROUP_M * tiles_n)) % gsz;
    const int tn = (bid % (GROUP_M * tiles_n)) / gsz;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
    const int wm = wave % WGM, wn = wave / WGM;
    const int kbeg = ws ? blockIdx.y * kper : 0;

    // loader: instruction q = t * NWAVES + wave of a tile moves 16 rows x 64 B (q < BM/16: A rows, else B
    // rows); lane -> row lane/4, LDS chunk lane%4 holding global chunk (lane%4) ^ ((row>>2)&3).  Buffer
    // loads with LDS destination: the per-lane byte offset is fixed, the k offset travels in the scalar
    // offset, so a tile costs no vector ALU work; and, unlike the flat-encoded LDS loads, they do not make
    // the compiler turn every LDS wait into lgkmcnt(0).
    constexpr int TA = BM / 16 / NWAVES, TB1 = BN / 16 / NWAVES; // instructions per wave: A, one B matrix
    static_assert(BM / 16 % NWAVES == 0 && BN / 16 % NWAVES == 0 && TA + NB * TB1 == LPT, "loader split");
    const int lrow = lane / 4, lchunk = (lane & 3) ^ ((lane >> 4) & 3);
    const __amdgpu_buffer_rsrc_t rs_x =
        __builtin_amdgcn_make_buffer_rsrc((void *)x, 0, ((T - 1) * ldx + K) * (int)sizeof(half_t), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void *)w, 0, N * K * (int)sizeof(half_t), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_w2 =
        __builtin_amdgcn_make_buffer_rsrc((void *)(NB == 2 ? w2 : w), 0, N * K * (int)sizeof(half_t), 0x00020000);
    // fixed bound: an array whose size depends on the template arguments, captured by the lambdas below, makes
    // this compiler drop the host stub of the kernel without a diagnostic
    static_assert(LPT <= 16, "goff");
    uint32_t goff[16];
#pragma unroll
    for (int t = 0; t < LPT; ++t) {
        const int q = wave + t * NWAVES;
        if (t < TA) {
            int ar = m0 + q * 16 + lrow;
            ar = ar < T ? ar : T - 1;
            goff[t] = ((uint32_t)ar * (uint32_t)ldx + kbeg + lchunk * 8) * 2u;
        } else {
            int br = n0 + (q - BM / 16) * 16 + lrow - (t >= TA + TB1 ? BN : 0);
            br = br < N ? br : N - 1;
            goff[t] = ((uint32_t)br * (uint32_t)K + kbeg + lchunk * 8) * 2u;
        }
    }
    auto issue_one = [&](int kt, int t) {
        half_t *st = lds + (kt % STAGES) * STAGE_HALVES;
        const uint32_t k0 = (uint32_t)kt * DMA_BK * 2u;
        auto dst = DMA_LP(st + (wave + t * NWAVES) * 16 * DMA_BK);
        if (t < TA) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, dst, 16, goff[t], k0, 0, 0);
        else if (t < TA + TB1) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, dst, 16, goff[t], k0, 0, 0);
        else __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w2, dst, 16, goff[t], k0, 0, 0);
    };
    auto issue = [&](int kt) {
#pragma unroll
        for (int t = 0; t < LPT; ++t) issue_one(kt, t);
    };

    const int frow = lane % 32, sw = (frow >> 2) & 3;
    int a_off[2], b_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const int pc = (ks * 2 + lane / 32) ^ sw;
        a_off[ks] = (wm * WTM + frow) * DMA_BK + pc * 8;
        b_off[ks] = BM * DMA_BK + ((NB == 1 ? wn * 128 : wn * 64) + frow) * DMA_BK + pc * 8;
    }
    half8_t af[2][FM], bf[2][4];
    auto lfrag = [&](int set, int kt, int ks) {
        const half_t *st = lds + (kt % STAGES) * STAGE_HALVES;
#pragma unroll
        for (int i = 0; i < FM; ++i) af[set][i] = load8(st + a_off[ks] + i * 32 * DMA_BK);
#pragma unroll
        for (int f = 0; f < 4; ++f) {
            const int roff = NB == 1 ? f * 32 : (f / 2) * BN + (f % 2) * 32;
            bf[set][f] = load8(st + b_off[ks] + roff * DMA_BK);
        }
    };

    float16_t acc[4][FM];
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[f][i][e] = 0.f;
    auto mma = [&](int set) {
#pragma unroll
        for (int f = 0; f < 4; ++f)
#pragma unroll
            for (int i = 0; i < FM; ++i)
                acc[f][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[set][f], af[set][i], acc[f][i], 0, 0, 0);
    };

    const int nk = (ws ? kper : K) / DMA_BK;
#pragma unroll
    for (int t = 0; t < AHEAD + (PREF ? 1 : 0); ++t)
        if (t < nk) issue(t);
    // tiles issued so far: min(nk, AHEAD); tiles kt+1 .. kt+AHEAD-1 are in flight at the top of iteration kt
    static_assert(!PREF, "the read-ahead pipeline lives in gemm_dma64_kernel");
    for (int kt = 0; kt < nk; ++kt) {
        // tile kt landed?  loads issued after it: tiles kt+1 .. min(kt+AHEAD-1, nk-1)
        const int last = kt + AHEAD - 1 < nk - 1 ? kt + AHEAD - 1 : nk - 1;
        const int beyond = last - kt;
        dma_wait_tiles<LPT, AHEAD - 1>(beyond);
        if (kt + AHEAD < nk) issue(kt + AHEAD);
        lfrag(0, kt, 0);
        lfrag(1, kt, 1);
        __builtin_amdgcn_sched_barrier(0);
        mma(0);
        mma(1);
        __builtin_amdgcn_sched_barrier(0);
    }

    const int mrow = lane % 32, ncol0 = 4 * (lane / 32);
    if (ws) {
        // slice z holds NB planes of [T][N] fp32: the plain product, or gate then up
        float *wz = ws + (size_t)blockIdx.y * NB * T * N;
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            const int m = m0 + wm * WTM + i * 32 + mrow;
#pragma unroll
            for (int f = 0; f < 4; ++f)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int j = NB == 1 ? f : f % 2, plane = NB == 1 ? 0 : f / 2;
                    const int n = n0 + (NB == 1 ? wn * 128 : wn * 64) + j * 32 + ncol0 + 8 * g;
                    float4_t o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = acc[f][i][4 * g + e];
                    if (m < T && n < N) *reinterpret_cast<float4_t *>(wz + ((size_t)plane * T + m) * N + n) = o;
                }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        const int m = m0 + wm * WTM + i * 32 + mrow;
        const int mc = m < T ? m : T - 1;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int nb = n0 + (NB == 1 ? wn * 128 : wn * 64) + j * 32 + ncol0;
            half4_t rv[4];
            if (NB == 1 && res) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    int n = nb + 8 * g;
                    n = n < N ? n : N - 4;
                    rv[g] = *reinterpret_cast<const half4_t *>(res + (size_t)mc * ldr + n);
                }
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = nb + 8 * g;
                half4_t o;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (NB == 2) o[e] = swiglu_to_half(acc[j][i][4 * g + e], acc[2 + j][i][4 * g + e]);
                    else if (res) o[e] = (half_t)((float)(half_t)acc[j][i][4 * g + e] + (float)rv[g][e]);
                    else o[e] = (half_t)acc[j][i][4 * g + e];
                }
                if (m < T && n < N) *reinterpret_cast<half4_t *>(out + (size_t)m * ldo + n) = o;
            }
        }
    }
}

#define DMA64_BK 64
// 256 x 256 tile, BK = 64, four waves of 128 x 128, on v_mfma_f32_16x16x32_f16 (64 accumulators of 4 registers
// per wave).  With operands that toggle like activations and weights this instruction sustains about 13 % more
// flops under the board's power limit than v_mfma_f32_32x32x16_f16 (it moves a fifth fewer register bytes per
// flop: the accumulator traffic halves).  A step is two sub-steps of 64 MFMAs on alternating fragment sets (8
// activation and 8 weight fragments each, read during the sub-step before); the workgroup barrier sits between
// the two: by then every wave has read the last fragments of the current stage and the next tile (issued
// during the previous step's second sub-step, one load behind every fourth MFMA) must have landed.
template <int NB>
__global__ __launch_bounds__(256, 1) void gemm_dma64_kernel(const half_t *__restrict__ x, int ldx, const half_t *__restrict__ w,
                                                           const half_t *__restrict__ w2, const half_t *res, int ldr,
                                                           half_t *out, int ldo, int T, int N, int K, int tiles_m,
                                                           int tiles_n) {
    constexpr int WTM = 128, BM = 256, BROWS = 256, BN = BROWS / NB;
    constexpr int STAGE_HALVES = (BM + BROWS) * DMA64_BK;
    constexpr int LPT = (BM + BROWS) / 8 / 4; // 16 load instructions per wave per tile
    constexpr int TA = BM / 8 / 4, TB1 = BN / 8 / 4;
    static_assert(TA + NB * TB1 == LPT, "loader split");
    extern __shared__ __attribute__((aligned(16))) half_t lds[];

    const int nblk = tiles_m * tiles_n;
    int bid = blockIdx.x;
    {
        const int per = nblk / 8;
        if (per > 0 && bid < per * 8) bid = (bid % 8) * per + bid / 8;
    }
    constexpr int GROUP_M = 8;
    const int group = bid / (GROUP_M * tiles_n);
    const int first_m = group * GROUP_M;
    const int gsz = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
    const int tm = first_m + (bid % (GROUP_M * tiles_n)) % gsz;
    const int tn = (bid % (GROUP_M * tiles_n)) / gsz;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
    const int wm = wave % 2, wn = wave / 2;

    const __amdgpu_buffer_rsrc_t rs_x =
        __builtin_amdgcn_make_buffer_rsrc((void *)x, 0, ((T - 1) * ldx + K) * (int)sizeof(half_t), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void *)w, 0, N * K * (int)sizeof(half_t), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_w2 =
        __builtin_amdgcn_make_buffer_rsrc((void *)(NB == 2 ? w2 : w), 0, N * K * (int)sizeof(half_t), 0x00020000);
    uint32_t goff[16];
#pragma unroll
    for (int t = 0; t < LPT; ++t) {
        const int q = wave + t * 4;
        const int srow = q * 8 + lane / 8; // row inside the stage
        const int gch = (lane & 7) ^ ((srow >> 1) & 7);
        if (t < TA) {
            int ar = m0 + srow;
            ar = ar < T ? ar : T - 1;
            goff[t] = (__umul24((unsigned)ar, (unsigned)ldx) + (unsigned)(gch * 8)) * 2u;
        } else {
            int br = n0 + (srow - BM) - (t >= TA + TB1 ? BN : 0);
            br = br < N ? br : N - 1;
            goff[t] = (__umul24((unsigned)br, (unsigned)K) + (unsigned)(gch * 8)) * 2u;
        }
    }
    auto issue_one = [&](int kt, int t) {
        half_t *st = lds + (kt & 1) * STAGE_HALVES;
        const uint32_t k0 = (uint32_t)kt * DMA64_BK * 2u;
        auto dst = DMA_LP(st + (wave + t * 4) * 8 * DMA64_BK);
        if (t < TA) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, dst, 16, goff[t], k0, 0, 0);
        else if (t < TA + TB1) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, dst, 16, goff[t], k0, 0, 0);
        else __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w2, dst, 16, goff[t], k0, 0, 0);
    };

    // fragment of a 16-row block for k-step ks (32 k): lane -> row lane%16, 16-byte chunk 4 ks + lane/16
    const int frow = lane % 16, sw = frow >> 1;
    int a_off[2], b_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const int pc = (ks * 4 + lane / 16) ^ sw;
        a_off[ks] = (wm * WTM + frow) * DMA64_BK + pc * 8;
        b_off[ks] = BM * DMA64_BK + ((NB == 1 ? wn * 128 : wn * 64) + frow) * DMA64_BK + pc * 8;
    }
    half8_t af[2][8], bf[2][8];
    auto one_read = [&](int set, int kt, int ks, int r) {
        const half_t *st = lds + (kt & 1) * STAGE_HALVES;
        if (r < 8) af[set][r] = load8(st + a_off[ks] + r * 16 * DMA64_BK);
        else {
            const int f = r - 8;
            const int roff = NB == 1 ? f * 16 : (f / 4) * BN + (f % 4) * 16;
            bf[set][f] = load8(st + b_off[ks] + roff * DMA64_BK);
        }
    };

    float4_t acc[8][8]; // [weight block][activation block]
#pragma unroll
    for (int f = 0; f < 8; ++f)
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[f][i][e] = 0.f;

    const int nk = K / DMA64_BK;
#pragma unroll
    for (int t = 0; t < LPT; ++t) issue_one(0, t);
    if (nk > 1) {
#pragma unroll
        for (int t = 0; t < LPT; ++t) issue_one(1, t);
        asm volatile("s_waitcnt vmcnt(16)\n\ts_barrier" ::: "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) one_read(0, 0, 0, r);

    // 64 MFMAs on fragment set `set`; behind MFMA i: one LDS read of the next fragments (every second MFMA, 16 in
    // all, weight fragment 0 and the activation fragments first: the order of use) and, in a sub-step that issues
    // a tile, one tile load behind every fourth MFMA
    auto substep = [&](int set, int next_kt, int next_ks, auto with_issue, int issue_kt) {
#pragma unroll
        for (int i = 0; i < 64; ++i) {
            const int f = i / 8, m = i % 8;
            // as text, accumulator tied to itself: with the builtin the register allocator moves the 64
            // accumulators between the two register files around the MFMAs (hundreds of copies per step)
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[f][m]) : "v"(bf[set][f]), "v"(af[set][m]));
            if ((i & 1) == 0) {
                const int r = i / 2; // 0..31: 16 reads in the first half of the sub-step
                if (r < 16) one_read(set ^ 1, next_kt, next_ks, r == 0 ? 8 : (r <= 8 ? r - 1 : r));
            }
            if (decltype(with_issue)::value && (i & 3) == 3) issue_one(issue_kt, i / 4);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    int kt = 0;
    for (; kt + 2 < nk; ++kt) {
        substep(0, kt, 1, std::false_type{}, 0);
        // every wave holds the last fragments of this stage; the next tile has landed
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        substep(1, kt + 1, 0, std::true_type{}, kt + 2);
    }
    for (; kt < nk; ++kt) {
        substep(0, kt, 1, std::false_type{}, 0);
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        substep(1, kt + 1, 0, std::false_type{}, 0); // past the last tile: reads a stage nobody uses
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); // the compiler does not see the MFMAs' result latency

    // lane l of a 16 x 16 block holds activation row l%16 and weight rows 4 (l/16) .. + 3: four output columns
    const int mrow = lane % 16, ncol0 = 4 * (lane / 16);
    auto product = [&](int j, int i) { // the four fp16 results of weight block j, activation block i
        half4_t h;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (NB == 2) h[e] = swiglu_to_half(acc[j][i][e], acc[4 + j][i][e]);
            else h[e] = (half_t)acc[j][i][e];
        }
        return h;
    };
    // Wide form (every row of out and res 16-byte aligned): the lanes of rows 0/1 and 2/3 of the wave swap the
    // results of two neighbouring weight blocks (v_permlane16_swap), after which a lane holds eight consecutive
    // columns: 16-byte stores and residual loads that cover 64 contiguous bytes of a row per instruction instead
    // of 8-byte ones that cover 32.  Same values, same roundings.
    const bool wide = ((uintptr_t)out & 15u) == 0 && ldo % 8 == 0 && N % 8 == 0 &&
                      (!(NB == 1 && res) || (((uintptr_t)res & 15u) == 0 && ldr % 8 == 0));
    if (wide) {
        const int g = lane / 16;
        // The residual values of the whole tile are asked for before the first store: out may be res itself (the
        // engine adds in place), so a load inside the store loop would have to wait behind the store before it,
        // one trip to memory per 16 bytes.  A thread reads exactly the elements it writes, so reading them all
        // first is the same computation.
        half8_t rv_all[NB == 1 ? 8 : 1][NB == 1 ? 4 : 1];
        if (NB == 1 && res) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int m = m0 + wm * WTM + i * 16 + mrow;
                const int mc = m < T ? m : T - 1;
#pragma unroll
                for (int jp = 0; jp < 4; ++jp) {
                    const int n = n0 + wn * 128 + 16 * (2 * jp + (g & 1)) + 8 * (g >> 1);
                    const int nc = n < N ? n : N - 8;
                    rv_all[NB == 1 ? i : 0][NB == 1 ? jp : 0] = load8(res + (size_t)mc * ldr + nc);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int m = m0 + wm * WTM + i * 16 + mrow;
#pragma unroll
            for (int jp = 0; jp < 4 / NB; ++jp) {
                const uint2_t a = __builtin_bit_cast(uint2_t, product(2 * jp, i));
                const uint2_t b = __builtin_bit_cast(uint2_t, product(2 * jp + 1, i));
                // odd rows of the first operand <-> even rows of the second
                const auto s0 = __builtin_amdgcn_permlane16_swap(a[0], b[0], false, false);
                const auto s1 = __builtin_amdgcn_permlane16_swap(a[1], b[1], false, false);
                const uint4_t packed = {s0[0], s1[0], s0[1], s1[1]};
                half8_t h = __builtin_bit_cast(half8_t, packed);
                const int n = n0 + (NB == 1 ? wn * 128 : wn * 64) + 16 * (2 * jp + (g & 1)) + 8 * (g >> 1);
                if (NB == 1 && res) {
                    const half8_t rv = rv_all[NB == 1 ? i : 0][NB == 1 ? jp : 0];
#pragma unroll
                    for (int e = 0; e < 8; ++e) h[e] = (half_t)((float)h[e] + (float)rv[e]);
                }
                if (m < T && n < N) store8(out + (size_t)m * ldo + n, h);
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int m = m0 + wm * WTM + i * 16 + mrow;
        const int mc = m < T ? m : T - 1;
#pragma unroll
        for (int j = 0; j < 8 / NB; ++j) {
            const int n = n0 + (NB == 1 ? wn * 128 : wn * 64) + j * 16 + ncol0;
            half4_t o = product(j, i);
            if (NB == 1 && res) {
                const int nc = n < N ? n : N - 4;
                const half4_t rv = *reinterpret_cast<const half4_t *>(res + (size_t)mc * ldr + nc);
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (half_t)((float)o[e] + (float)rv[e]);
            }
            if (m < T && n < N) *reinterpret_cast<half4_t *>(out + (size_t)m * ldo + n) = o;
        }
    }
}

template <int NB>
static int gemm_dma64_launch(const half_t *x, int ldx, const half_t *w, const half_t *w2, const half_t *res, int ldr,
                            half_t *out, int ldo, int T, int N, int K, hipStream_t s) {
    constexpr int BM = 256, BN = 256 / NB;
    const int tiles_m = (T + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const size_t smem = sizeof(half_t) * (size_t)2 * (BM + 256) * DMA64_BK;
    auto kern = gemm_dma64_kernel<NB>;
    static std::atomic<uint64_t> attr_done{0};
    int rc = llm_ensure_max_smem((const void *)kern, smem, attr_done);
    if (rc != LLM_OK) return rc;
    kern<<<dim3(tiles_m * tiles_n), dim3(256), smem, s>>>(x, ldx, w, w2, res, ldr, out, ldo, T, N, K, tiles_m, tiles_n);
    LLM_LAUNCH_CHECK("gemm_dma64_kernel");
    return LLM_OK;
}

// out[m][n] = finish(sum over z of ws[z][m][n]) (NB = 2: SiLU(sum of gate slices) * sum of up slices):
// four columns per thread, slices added in ascending z
template <int NB>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ ws, int S, int T, int N,
                                                            const half_t *res, int ldr, half_t *out, int ldo) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; // index of a group of four columns
    const int n4 = N / 4;
    if (i >= (size_t)T * n4) return;
    const int m = (int)(i / n4), n = (int)(i % n4) * 4;
    float4_t a[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) a[b] = *reinterpret_cast<const float4_t *>(ws + ((size_t)b * T + m) * N + n);
    for (int z = 1; z < S; ++z)
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const float4_t v = *reinterpret_cast<const float4_t *>(ws + (((size_t)z * NB + b) * T + m) * N + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) a[b][e] += v[e];
        }
    half4_t r = {0, 0, 0, 0}, o;
    if (NB == 1 && res) r = *reinterpret_cast<const half4_t *>(res + (size_t)m * ldr + n);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (NB == 2) o[e] = swiglu_to_half(a[0][e], a[NB - 1][e]);
        else o[e] = res ? (half_t)((float)(half_t)a[0][e] + (float)r[e]) : (half_t)a[0][e];
    }
    *reinterpret_cast<half4_t *>(out + (size_t)m * ldo + n) = o;
}

// fp32 partial tiles of split-K launches: one 64 MB buffer per (device, stream), so that launches on
// different streams never share partial sums.  llm_init allocates the default stream's buffer; any
// other stream gets its own at its first split-K launch (these run at 17..1024 rows, never inside a
// captured decode step) and gives it back in llm_stream_destroy.  Without a buffer (allocation failed, or the
// stream's first split-K launch falls inside a graph capture, where nothing may be allocated) the launch runs
// unsplit: same results up to summation order, fewer workgroups; g_unsplit_fallbacks counts those launches so
// that a slow prompt pass can be traced to them (llm_linear_unsplit_fallbacks).
static const size_t SPLITK_WS_BYTES = (size_t)64 << 20;
static std::atomic<long> g_unsplit_fallbacks{0};
struct SplitkWs {
    int device;
    hipStream_t stream;
    float *ptr;
};
static std::mutex g_splitk_mutex;
static std::vector<SplitkWs> g_splitk_ws;

static float *splitk_ws_for(hipStream_t s) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lock(g_splitk_mutex);
    for (const SplitkWs &e : g_splitk_ws)
        if (e.device == dev && e.stream == s) return e.ptr;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (s && hipStreamIsCapturing(s, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone) return nullptr;
    float *p = nullptr;
    if (hipMalloc((void **)&p, SPLITK_WS_BYTES) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    g_splitk_ws.push_back({dev, s, p});
    return p;
}

int gemm_init_workspace() {
    if (!splitk_ws_for(nullptr)) {
        llm_set_error("llm_init: no memory for the split-K workspace");
        return LLM_ERR_HIP;
    }
    return LLM_OK;
}

// llm_stream_destroy: the stream's work has finished, its buffer goes back
void gemm_release_workspace(hipStream_t s) {
    std::lock_guard<std::mutex> lock(g_splitk_mutex);
    for (size_t i = 0; i < g_splitk_ws.size(); ++i) {
        if (g_splitk_ws[i].stream != s || s == nullptr) continue;
        (void)hipFree(g_splitk_ws[i].ptr);
        g_splitk_ws.erase(g_splitk_ws.begin() + (long)i);
        --i;
    }
}

template <int NB, int WGM, int WGN, int STAGES, bool PREF, int OCC, int FM = 2>
static int gemm_dma_launch(const half_t *x, int ldx, const half_t *w, const half_t *w2, const half_t *res, int ldr,
                           half_t *out, int ldo, int T, int N, int K, int splits, hipStream_t s) {
    constexpr int BM = WGM * FM * 32, BN = WGN * 128 / NB;
    const int tiles_m = (T + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const size_t smem = sizeof(half_t) * (size_t)STAGES * (BM + WGN * 128) * DMA_BK;
    auto kern = gemm_dma_kernel<NB, WGM, WGN, STAGES, PREF, OCC, FM>;
    static std::atomic<uint64_t> attr_done{0};
    int rc = llm_ensure_max_smem((const void *)kern, smem, attr_done);
    if (rc != LLM_OK) return rc;
    float *ws = splits > 1 ? splitk_ws_for(s) : nullptr;
    if (splits > 1 && !ws) {
        splits = 1;
        g_unsplit_fallbacks.fetch_add(1, std::memory_order_relaxed);
    }
    if (splits > 1) {
        kern<<<dim3(tiles_m * tiles_n, splits), dim3(WGM * WGN * 64), smem, s>>>(x, ldx, w, w2, nullptr, 0, out, ldo, T, N, K,
                                                                               tiles_m, tiles_n, ws, K / splits);
        LLM_LAUNCH_CHECK("gemm_dma_kernel (split-K)");
        const size_t groups = (size_t)T * (N / 4);
        splitk_reduce_kernel<NB><<<dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, s>>>(ws, splits, T, N, res, ldr, out, ldo);
        LLM_LAUNCH_CHECK("splitk_reduce_kernel");
        return LLM_OK;
    }
    kern<<<dim3(tiles_m * tiles_n), dim3(WGM * WGN * 64), smem, s>>>(x, ldx, w, w2, res, ldr, out, ldo, T, N, K, tiles_m,
                                                                      tiles_n, nullptr, 0);
    LLM_LAUNCH_CHECK("gemm_dma_kernel");
    return LLM_OK;
}

// Number of k-slices for a launch with `tiles` output tiles: enough workgroups to put two on every CU,
// slices of at least 256 k that divide K into multiples of DMA_BK, partial tiles that fit the workspace.
static int pick_splits(long tiles, int T, int N, int K, int planes = 1) {
    int s = 1;
    while (s < 8 && tiles * s < 256 && K % (2 * s * DMA_BK) == 0 && K / (2 * s) >= 256 &&
           (size_t)(2 * s) * planes * T * N * sizeof(float) <= SPLITK_WS_BYTES)
        s *= 2;
    return s;
}

// ---------------------------------------------------------------------------
static int check_linear(const void *x, int ldx, const void *w, const void *out, int ldo, int T, int N, int K,
                        const char *who) {
    LLM_REQUIRE(x && w && out, "%s: null pointer", who);
    LLM_REQUIRE(T >= 0 && N > 0 && K > 0, "%s: T=%d N=%d K=%d", who, T, N, K);
    LLM_REQUIRE(K % 64 == 0, "%s: K=%d must be a multiple of 64", who, K);
    LLM_REQUIRE(N % 16 == 0, "%s: N=%d must be a multiple of 16", who, N);
    LLM_REQUIRE(ldx >= K && ldx % 8 == 0 && ldo >= N, "%s: ldx=%d ldo=%d", who, ldx, ldo);
    LLM_REQUIRE(aligned16(x) && aligned16(w), "%s: x and w must be 16-byte aligned", who);
    return LLM_OK;
}

// the direct-to-LDS kernels store (and read the residual) four halves at a time
// the tiles are fetched with 32-bit byte offsets into x and w
static bool dma_ok(const half_t *out, int ldo, const half_t *res, int ldr, int T, int ldx, int N, int K) {
    const size_t lim = (size_t)1 << 31;
    return ((uintptr_t)out & 7u) == 0 && ldo % 4 == 0 && (!res || (((uintptr_t)res & 7u) == 0 && ldr % 4 == 0)) &&
           (size_t)T * ldx * sizeof(half_t) < lim && (size_t)N * K * sizeof(half_t) < lim;
}

extern "C" {

long llm_linear_unsplit_fallbacks(void) { return g_unsplit_fallbacks.load(std::memory_order_relaxed); }

int llm_linear(const uint16_t *x, int ldx, const uint16_t *w, const uint16_t *residual, int ldr, uint16_t *out,
               int ldo, int T, int N, int K, llm_stream_t stream) {
    int rc = check_linear(x, ldx, w, out, ldo, T, N, K, "llm_linear");
    if (rc != LLM_OK) return rc;
    LLM_REQUIRE(!residual || ldr >= N, "llm_linear: ldr=%d", ldr);
    if (T == 0) return LLM_OK;
    hipStream_t s = (hipStream_t)stream;
    const half_t *xp = (const half_t *)x, *wp = (const half_t *)w, *rp = (const half_t *)residual;
    half_t *op = (half_t *)out;
    if (T == 1) return gemv_launch(xp, nullptr, 0.0, wp, rp, op, N, K, s);
    if (T <= 16 && skd_fits(N, K) && K % (4 * SKD_CHUNK) == 0 && aligned16(xp) && ldx % 8 == 0)
        return skinny_dma_launch<false, 4, 1, true>(xp, ldx, wp, nullptr, rp, ldr, op, ldo, T, N, K, s);
    if (T <= 16 && K % (SK_WAVES * 32) == 0) {
        skinny_kernel<false><<<dim3((N + 15) / 16), dim3(SK_WAVES * 64), 0, s>>>(xp, ldx, wp, nullptr, rp, ldr, op,
                                                                               ldo, T, N, K);
        LLM_LAUNCH_CHECK("skinny_kernel");
        return LLM_OK;
    }
    if (!dma_ok(op, ldo, rp, ldr, T, ldx, N, K) || N < 128) {
        if (T <= 64 || N < 256) return gemm_launch<64, 64, 2, 2, 1>(xp, ldx, wp, nullptr, rp, ldr, op, ldo, T, N, K, s);
        return gemm_launch<128, 128, 2, 2, 1>(xp, ldx, wp, nullptr, rp, ldr, op, ldo, T, N, K, s);
    }
    if (T <= 128) {
        // weight-streaming regime: 128 x 128 tiles, k split so that every CU has work
        const long tiles = (long)((N + 127) / 128);
        if (T <= 64) // 64-row tiles: half the x traffic of the 128-row tile
            return gemm_dma_launch<1, 2, 1, 4, false, 2, 1>(xp, ldx, wp, nullptr, rp, ldr, op, ldo, T, N, K,
                                                            pick_splits(tiles, T, N, K), s);
        // four waves of 32 rows rather than two of 64: with so few workgroups the MFMA work needs the SIMDs
        return gemm_dma_launch<1, 4, 1, 4, false, 2, 1>(xp, ldx, wp, nullptr, rp, ldr, op, ldo, T, N, K,
                                                        pick_splits(tiles, T, N, K), s);
    }
    // Measured at the 8B shapes: once the 256 x 256 tiles cover about three quarters of the CUs the
    // 4-wave tile below with its pinned, interleaved pipeline wins; with fewer tiles the 256 x 128 tile,
    // two workgroups per CU and a k split where that fills the chip.
    const long tiles = (long)((T + 255) / 256) * ((N + 255) / 256);
    if (tiles < 192) {
        const long t4 = (long)((T + 255) / 256) * ((N + 127) / 128);
        return gemm_dma_launch<1, 4, 1, 3, false, 2>(xp, ldx, wp, nullptr, rp, ldr, op, ldo, T, N, K,
                                                     pick_splits(t4, T, N, K), s);
    }
    // 256 x 256 tile as four waves of 128 x 128 (one per SIMD, accumulators in the second register
    // file): a third fewer LDS reads per MFMA than eight waves of 64 x 128, which on this
    // power-limited part is worth 3-12 % with real (non-constant) operands; BK = 64 so that tile loads
    // fetch whole cache lines
    return gemm_dma64_launch<1>(xp, ldx, wp, nullptr, rp, ldr, op, ldo, T, N, K, s); // K % 64 == 0 was checked
}

int llm_linear_swiglu(const uint16_t *x, int ldx, const uint16_t *wgate, const uint16_t *wup, uint16_t *out,
                      int ldo, int T, int N, int K, llm_stream_t stream) {
    int rc = check_linear(x, ldx, wgate, out, ldo, T, N, K, "llm_linear_swiglu");
    if (rc != LLM_OK) return rc;
    LLM_REQUIRE(wup && aligned16(wup), "llm_linear_swiglu: wup");
    if (T == 0) return LLM_OK;
    hipStream_t s = (hipStream_t)stream;
    const half_t *xp = (const half_t *)x, *gp = (const half_t *)wgate, *up = (const half_t *)wup;
    half_t *op = (half_t *)out;
    if (T == 1) return gemv_swiglu_launch(xp, nullptr, 0.0, gp, up, op, N, K, s);
    if (T <= 16 && skd_fits(N, K) && K % (4 * SKD_CHUNK) == 0)
        // x straight into registers here: with two weight tiles per slot the LDS ring has no room for x
        return skinny_dma_launch<true, 4, 1, false>(xp, ldx, gp, up, nullptr, 0, op, ldo, T, N, K, s);
    if (T <= 16 && K % (SK_WAVES * 32) == 0) {
        skinny_kernel<true><<<dim3((N + 15) / 16), dim3(SK_WAVES * 64), 0, s>>>(xp, ldx, gp, up, nullptr, 0, op, ldo,
                                                                              T, N, K);
        LLM_LAUNCH_CHECK("skinny_kernel<swiglu>");
        return LLM_OK;
    }
    if (!dma_ok(op, ldo, nullptr, 0, T, ldx, N, K) || N < 64) {
        if (T <= 64 || N < 256) return gemm_launch<64, 64, 2, 2, 2>(xp, ldx, gp, up, nullptr, 0, op, ldo, T, N, K, s);
        return gemm_launch<128, 64, 2, 2, 2>(xp, ldx, gp, up, nullptr, 0, op, ldo, T, N, K, s);
    }
    // (splitting k here costs more in fp32 partial traffic than the extra workgroups return)
    if (T <= 64)
        return gemm_dma_launch<2, 2, 1, 4, false, 2, 1>(xp, ldx, gp, up, nullptr, 0, op, ldo, T, N, K,
                                                        pick_splits(2 * (long)((N + 63) / 64), T, N, K, 2), s);
    if (T <= 128)
        return gemm_dma_launch<2, 4, 1, 4, false, 2, 1>(xp, ldx, gp, up, nullptr, 0, op, ldo, T, N, K,
                                                        pick_splits(2 * (long)((N + 63) / 64), T, N, K, 2), s);
    if ((long)((T + 255) / 256) * ((N + 127) / 128) < 192)
        return gemm_dma_launch<2, 4, 1, 3, false, 2>(xp, ldx, gp, up, nullptr, 0, op, ldo, T, N, K, 1, s);
    return gemm_dma64_launch<2>(xp, ldx, gp, up, nullptr, 0, op, ldo, T, N, K, s);
}

int llm_norm_linear(const uint16_t *x, const uint16_t *gain, double eps, const uint16_t *w, uint16_t *out, int N, int K,
                    llm_stream_t stream) {
    LLM_REQUIRE(x && gain && w && out, "llm_norm_linear: null pointer");
    LLM_REQUIRE(N > 0 && K > 0, "llm_norm_linear: N=%d K=%d", N, K);
    LLM_REQUIRE(aligned16(x) && aligned16(gain) && aligned16(w), "llm_norm_linear: pointers must be 16-byte aligned");
    return gemv_launch((const half_t *)x, (const half_t *)gain, eps, (const half_t *)w, nullptr, (half_t *)out, N, K,
                       (hipStream_t)stream);
}

int llm_embed_norm_linear(const uint16_t *table, const int32_t *ids, const int32_t *ids_offset, int vocab, uint16_t *x_out,
                          const uint16_t *gain, double eps, const uint16_t *w, uint16_t *out, int N, int K,
                          llm_stream_t stream) {
    LLM_REQUIRE(table && ids && x_out && gain && w && out, "llm_embed_norm_linear: null pointer");
    LLM_REQUIRE(N > 0 && K > 0 && vocab > 0, "llm_embed_norm_linear: N=%d K=%d vocab=%d", N, K, vocab);
    LLM_REQUIRE(aligned16(table) && aligned16(gain) && aligned16(w) && aligned16(x_out),
                "llm_embed_norm_linear: pointers must be 16-byte aligned");
    return gemv_embed_launch((const half_t *)table, ids, ids_offset, vocab, (half_t *)x_out, (const half_t *)gain, eps,
                             (const half_t *)w, (half_t *)out, N, K, (hipStream_t)stream);
}

int llm_norm_linear_swiglu(const uint16_t *x, const uint16_t *gain, double eps, const uint16_t *wgate,
                           const uint16_t *wup, uint16_t *out, int N, int K, llm_stream_t stream) {
    LLM_REQUIRE(x && gain && wgate && wup && out, "llm_norm_linear_swiglu: null pointer");
    LLM_REQUIRE(N > 0 && K > 0, "llm_norm_linear_swiglu: N=%d K=%d", N, K);
    LLM_REQUIRE(aligned16(x) && aligned16(gain) && aligned16(wgate) && aligned16(wup),
                "llm_norm_linear_swiglu: pointers must be 16-byte aligned");
    return gemv_swiglu_launch((const half_t *)x, (const half_t *)gain, eps, (const half_t *)wgate,
                              (const half_t *)wup, (half_t *)out, N, K, (hipStream_t)stream);
}

} // extern "C"
