// Causal GQA attention for one new token over the fp16 KV cache, optionally
// with RoPE and the KV-cache append of that token folded in.
//
// Cache layout (per layer), chosen so that both passes stream contiguous
// memory per KV head:
//   K: [Hkv][max_pos][hd]   a position's hd values are contiguous  (scores = K . q)
//   V: [Hkv][hd][max_pos]   a dim's positions are contiguous       (out = V^T-rows . p)
//
// Grid (Hkv, y): a workgroup owns one KV head and serves all G = Hq/Hkv query
// heads of the group.  Up to 512 keys there is one span of positions: four
// workgroups per head each take a quarter of the head's dims (each recomputes
// the cheap scores, so none waits for another) and write the result directly.
// Beyond that workgroup y takes the 512-position span y with all dims, leaves
// (max, sum, unnormalised P.V), and the last workgroup of the head to finish
// (a self-resetting counter) merges the spans.  Both products run on the matrix
// pipe with fp16 operands and fp32 accumulation (the probabilities are rounded
// to fp16 like the prompt-pass kernel's); maxima, sums and the merge stay in fp32
// and only the final output is rounded (reference: src/inference/inference.cu:736-947,
// which keeps fp32 throughout; the difference is inside the 2e-2 the tests allow).
#include <cfloat>
#include <cmath>
#include <mutex>

#include "common.hpp"

#include "attn_decode_body.hpp"

template <int HD, int G, bool FUSED, int DSN>
__global__ __launch_bounds__(AD_THREADS) void attn_decode_kernel(const AdArgs a) {
    __shared__ float sc[G * AD_LS];
    __shared__ __attribute__((aligned(16))) half_t qs[G * HD];
    __shared__ __attribute__((aligned(16))) half_t knew[HD];
    __shared__ __attribute__((aligned(16))) half_t vnew[HD];
    __shared__ float s_m[G], s_l[G];
    __shared__ int s_last;
    int pos = a.pos_host + (a.pos_dev ? *a.pos_dev : 0);
    if (pos > a.max_pos - 1) pos = a.max_pos - 1;
    if (pos < 0) pos = 0;
    const int n_active = pos / AD_LS + 1;
    const int y = blockIdx.y;
    if (n_active == 1) {
        // one span: workgroups 0..DSN-1 of the head each take a slice of its dims and write
        // the result directly (no synchronisation between them)
        if (y >= DSN) return;
        attn_decode_body<HD, G, FUSED, HD / DSN, AD_LS>(a, sc, qs, knew, vnew, s_m, s_l, &s_last, pos, 1, 0,
                                                        y * (HD / DSN), y == 0);
    } else {
        // several spans: workgroup y takes span y with all dims; the last to finish merges
        if (y >= n_active) return;
        attn_decode_body<HD, G, FUSED, HD, AD_LS>(a, sc, qs, knew, vnew, s_m, s_l, &s_last, pos, n_active, y, 0,
                                                  y == n_active - 1);
    }
}

// ---------------------------------------------------------------------------
// Attention of one token and the projection that consumes it, in one launch.
//
// The attention above occupies Hkv * DSN workgroups for a few microseconds and moves about a megabyte:
// HBM idles meanwhile, and the output projection launched behind it then pays its own launch, its own
// first trip to HBM and the streaming of its whole matrix.  Here the workgroups with the lowest ids run
// the attention exactly as above; every other workgroup belongs to the projection: it asks for all of its
// weight rows at once (they stay in registers), and only then waits for the attention output, stages it
// in LDS and reduces.  Streaming the matrix thus overlaps the attention.
//
// Hand-over without counters or fences: the attention output buffer starts out filled with a 16-bit
// pattern that the attention never writes (AO_EMPTY, a NaN; a result with those bits is stored with the
// lowest bit cleared).  The attention stores its results write-through at device scope; the projection
// workgroups read the buffer with device-scope loads until no word holds the pattern any more: the data
// is its own flag.  The launch refills `next`, the buffer of the following launch in stream order (the
// host passes a ring of at least two buffers), so every launch finds its own buffer empty.
// One workgroup per CU at most (grid <= number of CUs), and workgroups are dispatched in id order, so the
// attention workgroups are running before any projection workgroup can wait for them: the wait cannot
// deadlock, also when launches of several streams share the device (each queue hands out its workgroups in
// id order, so a resident projection workgroup implies that its launch's attention workgroups were handed
// out before it).  It is bounded anyway (spin_limit rounds, AO_SPIN_LIMIT by default, after which the workgroup
// carries on with whatever the buffer holds and counts a timeout in *timeouts: the host must then treat the
// projection's output as invalid and redo the step).
// ---------------------------------------------------------------------------
#define AO_WAVES 8          // = AD_WAVES: both roles use 512 threads
#define AO_ROWS 3           // weight rows per wavefront of the projection part, at most
#define AO_KSTEPS 8         // 16-byte loads per lane and row: K <= 4096
#define AO_SPIN_LIMIT (1 << 18)
#define AO_EMPTY 0xFFFFu

struct AoArgs {
    const half_t *w;   // [N, K] projection weights
    const half_t *res; // [N] residual (may alias out) or null
    half_t *out;       // [N]
    uint16_t *next;    // [K] attention output buffer of the next launch: refilled with AO_EMPTY here
    int N, K;
    int n_owg;         // projection workgroups
    int rows;          // weight rows per wavefront (<= AO_ROWS)
    int *timeouts;     // waits that ran into the limit
    int spin_limit;    // polling rounds before a wait gives up
};

// The projection role of a launch some of whose workgroups produce the projection's input vector (a.out, handed
// over as described above): all weight rows of the workgroup are requested at once (ao_projection_loads), then the
// vector is polled for, staged in LDS and reduced against (ao_projection_finish).  n_attn: workgroups in front
// that take no rows.
struct AoRows {
    half8_t wreg[AO_ROWS][AO_KSTEPS];
    half_t resv[AO_ROWS];
};

// first half: the weight rows (and residual values) of this workgroup, all asked for at once
__device__ __forceinline__ void ao_projection_loads(const AoArgs &o, const int n_attn, const int head_start, AoRows &R) {
    const int wg = blockIdx.x, tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int K = o.K, N = o.N;
    // Row i of projection workgroup p is p + n_owg * i (adjacent workgroups read adjacent rows at the same time), dealt
    // to its wavefronts in turn: every workgroup, i.e. every CU, streams N / n_owg rows to within one (18 or 19 of the
    // 8B model's 4096 on 224 CUs), where rows dealt wavefront by wavefront over the whole launch left 24 to some CUs
    // and 16 to the others.
    const int wslot = (wg - n_attn) + o.n_owg * wave;
    const int wtotal = o.n_owg * AO_WAVES;
    // (attention + projection launch: a head start of a little under a microsecond for the attention's own loads,
    // measured per launch: 12.2 -> 11.4 us with the first version of the attention; against the current one three
    // pauses beat 0-2 and 4-8)
    for (int dl = 0; dl < head_start; ++dl) __builtin_amdgcn_s_sleep(8);
#pragma unroll
    for (int r = 0; r < AO_ROWS; ++r) {
        int row = wslot + wtotal * r;
        const bool live = r < o.rows && row < N;
        row = live ? row : N - 1;
#pragma unroll
        for (int j = 0; j < AO_KSTEPS; ++j) {
            const int k = lane * 8 + 512 * j;
            R.wreg[r][j] = (live && k < K) ? load8_nt(o.w + (size_t)row * K + k) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }
        R.resv[r] = (live && o.res) ? o.res[row] : (half_t)0.f;
    }
}

// second half: wait for the input vector (a.out, handed over as described above), stage it in xs (K halves of
// LDS), reduce the rows against it and store
__device__ __forceinline__ void ao_projection_finish(const AdArgs &a, const AoArgs &o, half_t *xs, const int n_attn, const AoRows &R) {
    const int wg = blockIdx.x, tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int K = o.K, N = o.N;
    const int wslot = (wg - n_attn) + o.n_owg * wave;
    const int wtotal = o.n_owg * AO_WAVES;
    // ---- the attention output, as soon as it is there ------------------------------------
    {
        const uint32_t *src = reinterpret_cast<const uint32_t *>(a.out);
        uint32_t *dst = reinterpret_cast<uint32_t *>(xs);
        // K/2 words over 512 threads: at most AO_KSTEPS/2 per thread, all asked for in one round
        constexpr int WPT = AO_KSTEPS * 512 / 2 / AD_THREADS;
        uint32_t v[WPT];
        int spins = 0;
        for (;;) {
            bool empty = false;
#pragma unroll
            for (int i = 0; i < WPT; ++i) {
                const int c = tid + AD_THREADS * i;
                v[i] = c < K / 2 ? __hip_atomic_load(src + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
            }
#pragma unroll
            for (int i = 0; i < WPT; ++i) empty |= (v[i] & 0xFFFFu) == AO_EMPTY || (v[i] >> 16) == AO_EMPTY;
            if (!empty) break;
            if (++spins > o.spin_limit) {
                atomicAdd(o.timeouts, 1);
                break;
            }
            __builtin_amdgcn_s_sleep(2);
        }
#pragma unroll
        for (int i = 0; i < WPT; ++i) {
            const int c = tid + AD_THREADS * i;
            if (c < K / 2) dst[c] = v[i];
        }
    }
    __syncthreads();
    // all rows of the wavefront against one read of the staged vector, then their reductions side by side
    float acc[AO_ROWS];
#pragma unroll
    for (int r = 0; r < AO_ROWS; ++r) acc[r] = 0.f;
#pragma unroll
    for (int j = 0; j < AO_KSTEPS; ++j) {
        const int k = lane * 8 + 512 * j;
        if (k < K) {
            const half8_t x = load8(xs + k);
#pragma unroll
            for (int r = 0; r < AO_ROWS; ++r) acc[r] = dot8(R.wreg[r][j], x, acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < AO_ROWS; ++r) acc[r] = wave_sum(acc[r]);
#pragma unroll
    for (int r = 0; r < AO_ROWS; ++r) {
        const int row = wslot + wtotal * r;
        if (lane == 0 && r < o.rows && row < N) {
            half_t h = (half_t)acc[r];
            if (o.res) h = (half_t)((float)h + (float)R.resv[r]); // the reference's add_norm on the stored projection
            o.out[row] = h;
        }
    }
}

// Arguments as scalars, what the attention workgroups need for their first loads in front (the first 14 dwords
// reach the wavefronts in scalar registers, see the build flags; structs passed by value do not).
// kvh_maxpos = n_kv_heads | max_pos << 8.
template <int HD, int G, int DSN>
__global__ __launch_bounds__(AD_THREADS) void attn_oproj_kernel(const int32_t *pos_dev, const half_t *qkv, half_t *kc,
                                                                half_t *vc, const float *table, const half_t *w,
                                                                int pos_host, int kvh_maxpos, half_t *attn_out,
                                                                const half_t *res, half_t *out, uint16_t *next, int N,
                                                                int K, int n_owg, int rows, int *timeouts, int spin_limit) {
    AdArgs a = {};
    a.q = qkv;
    a.kc = kc;
    a.vc = vc;
    a.out = attn_out;
    a.table = table;
    a.pos_host = pos_host;
    a.pos_dev = pos_dev;
    a.n_kv_heads = kvh_maxpos & 0xff;
    a.max_pos = (int)((unsigned)kvh_maxpos >> 8);
    a.splits = 1;
    const AoArgs o = {w, res, out, next, N, K, n_owg, rows, timeouts, spin_limit};
    __shared__ float sc[G * AD_LS];
    __shared__ __attribute__((aligned(16))) half_t qs[G * HD];
    __shared__ __attribute__((aligned(16))) half_t knew[HD];
    __shared__ __attribute__((aligned(16))) half_t vnew[HD];
    __shared__ float s_m[G], s_l[G];
    __shared__ int s_last;
    const int n_attn = a.n_kv_heads * DSN;
    const int wg = blockIdx.x, tid = threadIdx.x;
    if (wg < n_attn) {
        int pos = a.pos_host + (a.pos_dev ? *a.pos_dev : 0);
        if (pos > a.max_pos - 1) pos = a.max_pos - 1;
        if (pos > AD_LS - 1) pos = AD_LS - 1; // this form serves one span; the host picks it below AD_LS only
        if (pos < 0) pos = 0;
        const int kvh = wg % a.n_kv_heads, y = wg / a.n_kv_heads;
        attn_decode_body<HD, G, true, HD / DSN, AD_LS, true>(a, sc, qs, knew, vnew, s_m, s_l, &s_last, pos, 1, 0,
                                                                    y * (HD / DSN), y == 0, kvh);
        // off the critical path: the next launch's buffer back to "empty" (visible at the end of this kernel)
        uint32_t *nx = reinterpret_cast<uint32_t *>(o.next);
        for (int c = wg * AD_THREADS + tid; c < o.K / 2; c += n_attn * AD_THREADS) nx[c] = AO_EMPTY | (AO_EMPTY << 16);
        return;
    }
    AoRows R;
    ao_projection_loads(o, n_attn, 3, R);
    ao_projection_finish(a, o, reinterpret_cast<half_t *>(sc), n_attn, R); // K halves: K * 2 <= sizeof(sc), checked by the host
}

template <int HD, int G>
static int launch_attn_oproj(AdArgs a, AoArgs o, hipStream_t s) {
    constexpr int DSN = HD >= 128 ? 4 : 1;
    static_assert(AO_WAVES == AD_WAVES, "both roles share the workgroup size");
    LLM_REQUIRE((size_t)o.K * sizeof(half_t) <= sizeof(float) * G * AD_LS, "llm_attn_decode_rope_oproj: K=%d does not fit the staging buffer", o.K);
    int cus = 0;
    int rc = llm_cu_count_cached(&cus);
    if (rc != LLM_OK) return rc;
    const int n_attn = a.n_kv_heads * DSN;
    LLM_REQUIRE(cus > n_attn, "llm_attn_decode_rope_oproj: %d attention workgroups on %d CUs", n_attn, cus);
    // at most one workgroup per CU: all of them are resident at once
    int owg = (o.N + AO_WAVES - 1) / AO_WAVES;
    if (owg > cus - n_attn) owg = cus - n_attn;
    const int rows = (o.N + owg * AO_WAVES - 1) / (owg * AO_WAVES);
    LLM_REQUIRE(rows <= AO_ROWS, "llm_attn_decode_rope_oproj: N=%d needs %d rows per wavefront on %d CUs (at most %d)", o.N, rows,
                cus, AO_ROWS);
    o.n_owg = owg;
    o.rows = rows;
    a.splits = 1;
    LLM_REQUIRE(a.n_kv_heads < 256 && a.max_pos < (1 << 23), "llm_attn_decode_rope_oproj: %d kv heads, max_pos %d", a.n_kv_heads,
                a.max_pos);
    attn_oproj_kernel<HD, G, DSN><<<dim3(n_attn + owg), dim3(AD_THREADS), 0, s>>>(
        a.pos_dev, a.q, a.kc, a.vc, a.table, o.w, a.pos_host, a.n_kv_heads | (a.max_pos << 8), a.out, o.res, o.out, o.next, o.N,
        o.K, o.n_owg, o.rows, o.timeouts, o.spin_limit);
    LLM_LAUNCH_CHECK("attn_oproj_kernel");
    return LLM_OK;
}

template <int HD, int G, bool FUSED>
static int launch_decode(AdArgs a, void *ws, hipStream_t s) {
    constexpr int DSN = HD >= 128 ? 4 : 1;
    const int Hq = a.n_kv_heads * G;
    a.ws_acc = (float *)ws;
    a.ws_ml = a.ws_acc + (size_t)Hq * AD_MAX_SPLITS * HD;
    a.counters = (int *)(a.ws_ml + (size_t)Hq * AD_MAX_SPLITS * 2);
    const int splits = (a.max_pos + AD_LS - 1) / AD_LS;
    LLM_REQUIRE(splits <= AD_MAX_SPLITS, "llm_attn_decode: max_pos=%d exceeds %d", a.max_pos, AD_MAX_SPLITS * AD_LS);
    a.splits = splits;
    const int gy = splits > DSN ? splits : DSN;
    attn_decode_kernel<HD, G, FUSED, DSN><<<dim3(a.n_kv_heads, gy), dim3(AD_THREADS), 0, s>>>(a);
    LLM_LAUNCH_CHECK("attn_decode_kernel");
    return LLM_OK;
}

template <bool FUSED>
static int dispatch_decode(AdArgs a, int n_heads, int head_dim, void *ws, hipStream_t s) {
    const int G = n_heads / a.n_kv_heads;
#define AD_CASE(HD_, G_) \
    if (head_dim == HD_ && G == G_) return launch_decode<HD_, G_, FUSED>(a, ws, s);
    AD_CASE(128, 4)
    AD_CASE(128, 8)
    AD_CASE(128, 1)
    AD_CASE(64, 4)
    AD_CASE(64, 1)
    AD_CASE(32, 4)
    AD_CASE(32, 1)
#undef AD_CASE
    llm_set_error("llm_attn_decode: head_dim=%d with group size %d is not built", head_dim, G);
    return LLM_ERR_INVALID;
}

// ---------------------------------------------------------------------------
// Long contexts: two launches.  attn_span_kernel gives every (KV head, span of positions) its own
// workgroup (attn_span_wave: eight wavefronts of 32 positions, each on its own until the combine; two
// workgroups fit a CU) and leaves (max, sum, unnormalised P.V) per span; attn_merge_kernel, one workgroup
// per query head, combines them.  No fence, counter or last-workgroup tail: beyond a few spans that tail
// costs more than the second launch.
// ---------------------------------------------------------------------------
#define AD_MERGE_THREADS 512

// (arguments as leading scalars, like attn_oproj_kernel: kvh_maxpos = n_kv_heads | max_pos << 8,
// splits_target = splits | span_target << 16)
template <int HD, int G>
__global__ __launch_bounds__(AD_SPAN_THREADS, 4) void attn_span_kernel(const int32_t *pos_dev, const half_t *q, half_t *kc,
                                                                  half_t *vc, const float *table, int pos_host,
                                                                  int kvh_maxpos, int splits_target, float *ws_acc,
                                                                  float *ws_ml) {
    AdArgs a = {};
    a.q = q;
    a.kc = kc;
    a.vc = vc;
    a.table = table;
    a.n_kv_heads = kvh_maxpos & 0xff;
    a.max_pos = (int)((unsigned)kvh_maxpos >> 8);
    a.splits = splits_target & 0xffff;
    a.span_target = (int)((unsigned)splits_target >> 16);
    a.ws_acc = ws_acc;
    a.ws_ml = ws_ml;
    int pos = pos_host + (pos_dev ? *pos_dev : 0);
    if (pos > a.max_pos - 1) pos = a.max_pos - 1;
    if (pos < 0) pos = 0;
    const int span = ad_long_span(pos + 1, a.span_target);
    const int n_active = (pos + span) / span;
    const int y = blockIdx.y;
    if (y >= n_active) return;
    if (y == n_active - 1) attn_span_wave<HD, G, true>(a, pos, y, blockIdx.x, span);
    else attn_span_wave<HD, G, false>(a, pos, y, blockIdx.x, span);
}

// AGENT_OUT: the head's result leaves as 8-byte device-scope stores with the "not written yet" pattern avoided,
// for readers inside the same launch (merge_oproj_kernel).
template <int HD, int G, bool AGENT_OUT = false>
__device__ __forceinline__ void attn_merge_body(const AdArgs &a, const int h) {
    constexpr int PARTS = AD_MERGE_THREADS / HD;
    __shared__ float w[AD_MAX_SPLITS];
    __shared__ float red[2 * AD_MERGE_THREADS / 64];
    __shared__ float part_o[AD_MERGE_THREADS];
    __shared__ float s_M, s_L;
    int pos = a.pos_host + (a.pos_dev ? *a.pos_dev : 0);
    if (pos > a.max_pos - 1) pos = a.max_pos - 1;
    if (pos < 0) pos = 0;
    const int n = ad_long_spans(pos + 1, a.span_target);
    const int kvh = h / G, hh = h % G, splits = a.splits;
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    float m = -FLT_MAX, l = 0.f;
    if (tid < n) {
        const size_t b = ((size_t)kvh * splits + tid) * G + hh;
        m = a.ws_ml[b * 2];
        l = a.ws_ml[b * 2 + 1];
    }
    float mx = wave_max(m);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    if (tid == 0) {
        float t = red[0];
        for (int q = 1; q < AD_MERGE_THREADS / 64; ++q) t = fmaxf(t, red[q]);
        s_M = t;
    }
    __syncthreads();
    const float wgt = tid < n ? expf(m - s_M) : 0.f;
    if (tid < n) w[tid] = wgt;
    float ls = wave_sum(l * wgt);
    if (lane == 0) red[AD_MERGE_THREADS / 64 + wave] = ls;
    __syncthreads();
    if (tid == 0) {
        float t = 0.f;
        for (int q = 0; q < AD_MERGE_THREADS / 64; ++q) t += red[AD_MERGE_THREADS / 64 + q];
        s_L = t;
    }
    const int d = tid % HD, part = tid / HD;
    // four spans per round: their loads are independent, so a round costs one trip to memory
    float o = 0.f;
    const float *accp = a.ws_acc + ((size_t)kvh * splits * G + hh) * HD + d;
    int s = part;
    for (; s + 3 * PARTS < n; s += 4 * PARTS) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = accp[(size_t)(s + u * PARTS) * G * HD];
#pragma unroll
        for (int u = 0; u < 4; ++u) o += v[u] * w[s + u * PARTS];
    }
    for (; s < n; s += PARTS) o += accp[(size_t)s * G * HD] * w[s];
    part_o[tid] = o;
    __syncthreads();
    __shared__ __attribute__((aligned(8))) uint16_t res16[AGENT_OUT ? HD : 4];
    if (tid < HD) {
        float t = part_o[tid];
#pragma unroll
        for (int q = 1; q < PARTS; ++q) t += part_o[tid + q * HD];
        const half_t r = (half_t)(t / s_L);
        if (AGENT_OUT) {
            uint16_t bits = __builtin_bit_cast(uint16_t, r);
            if (bits == 0xFFFFu) bits = 0xFFFEu; // 0xFFFF marks "not written yet" for the reader
            res16[tid] = bits;
        } else {
            a.out[(size_t)h * HD + tid] = r;
        }
    }
    if (AGENT_OUT) {
        static_assert(HD % 4 == 0, "results are stored four at a time");
        __syncthreads();
        if (tid < HD / 4)
            __hip_atomic_store(reinterpret_cast<unsigned long long *>(a.out + (size_t)h * HD) + tid,
                               reinterpret_cast<const unsigned long long *>(res16)[tid], __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <int HD, int G>
__global__ __launch_bounds__(AD_MERGE_THREADS) void attn_merge_kernel(const AdArgs a) {
    attn_merge_body<HD, G>(a, blockIdx.x);
}

// Long form on the host: the span target of this device (a.span_target), the span count of the workspace layout
// (a.splits: never fewer than any position below max_pos uses) and the second grid dimension of the span kernel
// (the spans in use when the position is known here, else that same upper bound).
static int ad_long_setup(AdArgs &a, int *gy) {
    int cus = 0;
    int rc = llm_cu_count_cached(&cus);
    if (rc != LLM_OK) return rc;
    int target = cus / a.n_kv_heads;
    a.span_target = target < 1 ? 1 : target > 64 ? 64 : target;
    const int splits = ad_long_max_spans(a.max_pos, a.span_target);
    LLM_REQUIRE(splits <= AD_MAX_SPLITS, "decode attention: max_pos=%d exceeds %d", a.max_pos, AD_MAX_SPLITS * AD_SPAN);
    a.splits = splits;
    LLM_REQUIRE(a.n_kv_heads < 256 && a.max_pos < (1 << 23), "decode attention: %d kv heads, max_pos %d", a.n_kv_heads, a.max_pos);
    *gy = a.pos_dev ? splits : ad_long_spans(a.pos_host + 1, a.span_target);
    return LLM_OK;
}

template <int HD, int G>
static int launch_decode_long(AdArgs a, void *ws, hipStream_t s) {
    const int Hq = a.n_kv_heads * G;
    a.ws_acc = (float *)ws;
    a.ws_ml = a.ws_acc + (size_t)Hq * AD_MAX_SPLITS * HD;
    a.counters = nullptr;
    int gy = 0;
    int rc = ad_long_setup(a, &gy);
    if (rc != LLM_OK) return rc;
    attn_span_kernel<HD, G><<<dim3(a.n_kv_heads, gy), dim3(AD_SPAN_THREADS), 0, s>>>(
        a.pos_dev, a.q, a.kc, a.vc, a.table, a.pos_host, a.n_kv_heads | (a.max_pos << 8), a.splits | (a.span_target << 16), a.ws_acc,
        a.ws_ml);
    LLM_LAUNCH_CHECK("attn_span_kernel");
    attn_merge_kernel<HD, G><<<dim3(Hq), dim3(AD_MERGE_THREADS), 0, s>>>(a);
    LLM_LAUNCH_CHECK("attn_merge_kernel");
    return LLM_OK;
}

// ---------------------------------------------------------------------------
// Long contexts, merge and output projection in one launch.  The span kernel runs as above; in the second
// launch the first Hq workgroups merge one query head each and hand the result over to the projection
// workgroups exactly as the attention workgroups of attn_oproj_kernel do (same buffers, same polling,
// same refill of the next launch's buffer), so the projection's weights stream while the spans are merged
// and the projection needs no launch of its own.
// ---------------------------------------------------------------------------
template <int HD, int G>
__global__ __launch_bounds__(AD_THREADS) void merge_oproj_kernel(const int32_t *pos_dev, const float *ws_ml,
                                                                 const float *ws_acc, const half_t *w, int pos_host,
                                                                 int kvh_maxpos, int splits_target, int N, int K, int n_owg,
                                                                 half_t *attn_out, const half_t *res, half_t *out,
                                                                 uint16_t *next, int rows, int *timeouts, int spin_limit) {
    AdArgs a = {};
    a.out = attn_out;
    a.pos_host = pos_host;
    a.pos_dev = pos_dev;
    a.n_kv_heads = kvh_maxpos & 0xff;
    a.max_pos = (int)((unsigned)kvh_maxpos >> 8);
    a.splits = splits_target & 0xffff;
    a.span_target = (int)((unsigned)splits_target >> 16);
    a.ws_acc = const_cast<float *>(ws_acc);
    a.ws_ml = const_cast<float *>(ws_ml);
    const AoArgs o = {w, res, out, next, N, K, n_owg, rows, timeouts, spin_limit};
    static_assert(AD_MERGE_THREADS == AD_THREADS, "both roles share the workgroup size");
    __shared__ __attribute__((aligned(16))) half_t xs[AO_KSTEPS * 512];
    const int n_first = a.n_kv_heads * G;
    const int wg = blockIdx.x, tid = threadIdx.x;
    // (The merging workgroups take no projection rows: a wavefront's loads come back in order, so the reads of the
    // spans' partial results would stand behind its weight rows -- measured 1.7 us per launch slower.)
    if (wg < n_first) {
        attn_merge_body<HD, G, true>(a, wg);
        uint32_t *nx = reinterpret_cast<uint32_t *>(o.next);
        for (int c = wg * AD_THREADS + tid; c < o.K / 2; c += n_first * AD_THREADS) nx[c] = AO_EMPTY | (AO_EMPTY << 16);
        return;
    }
    AoRows R;
    ao_projection_loads(o, n_first, 0, R);
    ao_projection_finish(a, o, xs, n_first, R);
}

// projection workgroups and rows per wavefront behind n_first producer workgroups; false when they do not fit
static bool ao_partition(int N, int n_first, int cus, int *owg_out, int *rows_out) {
    if (cus <= n_first) return false;
    int owg = (N + AO_WAVES - 1) / AO_WAVES;
    if (owg > cus - n_first) owg = cus - n_first; // at most one workgroup per CU: all of them are resident at once
    const int rows = (N + owg * AO_WAVES - 1) / (owg * AO_WAVES);
    *owg_out = owg;
    *rows_out = rows;
    return rows <= AO_ROWS;
}

template <int HD, int G>
static int launch_long_oproj(AdArgs a, AoArgs o, void *ws, hipStream_t s) {
    const int Hq = a.n_kv_heads * G;
    int cus = 0;
    int rc = llm_cu_count_cached(&cus);
    if (rc != LLM_OK) return rc;
    LLM_REQUIRE(ao_partition(o.N, Hq, cus, &o.n_owg, &o.rows),
                "llm_attn_decode_rope_long_oproj: N=%d behind %d merge workgroups does not fit %d CUs", o.N, Hq, cus);
    a.ws_acc = (float *)ws;
    a.ws_ml = a.ws_acc + (size_t)Hq * AD_MAX_SPLITS * HD;
    a.counters = nullptr;
    int gy = 0;
    rc = ad_long_setup(a, &gy);
    if (rc != LLM_OK) return rc;
    attn_span_kernel<HD, G><<<dim3(a.n_kv_heads, gy), dim3(AD_SPAN_THREADS), 0, s>>>(
        a.pos_dev, a.q, a.kc, a.vc, a.table, a.pos_host, a.n_kv_heads | (a.max_pos << 8), a.splits | (a.span_target << 16), a.ws_acc,
        a.ws_ml);
    LLM_LAUNCH_CHECK("attn_span_kernel");
    merge_oproj_kernel<HD, G><<<dim3(Hq + o.n_owg), dim3(AD_THREADS), 0, s>>>(
        a.pos_dev, a.ws_ml, a.ws_acc, o.w, a.pos_host, a.n_kv_heads | (a.max_pos << 8), a.splits | (a.span_target << 16), o.N, o.K,
        o.n_owg, a.out, o.res, o.out, o.next, o.rows, o.timeouts, o.spin_limit);
    LLM_LAUNCH_CHECK("merge_oproj_kernel");
    return LLM_OK;
}

// ---------------------------------------------------------------------------
// Batched decode: B independent sequences (each with its own KV cache and position) in one launch;
// workgroup z serves sequence z with exactly the code of the single-sequence kernels.
// ---------------------------------------------------------------------------
#define AD_MAX_BATCH 16

struct AdBatch {
    const half_t *qkv; // [B][ldq] raw projection rows
    int ldq;
    half_t *out;       // [B][ldo]
    int ldo;
    half_t *kc[AD_MAX_BATCH], *vc[AD_MAX_BATCH];
    int pos[AD_MAX_BATCH];
    size_t ws_floats;  // workspace floats per sequence (long form)
};

// The caches and positions of the sequences in device memory (llm_batch_desc), read by the kernels when they run:
// what a captured launch needs, whose arguments cannot change from one replay to the next.
struct AdBatchDev {
    const llm_batch_desc *desc;
    size_t cache_offset; // elements from a sequence's cache pointers to the layer's part of the caches
};

__device__ __forceinline__ void ad_sequence_caches(const AdBatch &b, const AdBatchDev &, int z, AdArgs &a) {
    a.kc = b.kc[z];
    a.vc = b.vc[z];
    a.pos_host = b.pos[z];
}
__device__ __forceinline__ void ad_sequence_caches(const AdBatch &, const AdBatchDev &d, int z, AdArgs &a, int) {
    a.kc = reinterpret_cast<half_t *>(d.desc->k_cache[z]) + d.cache_offset;
    a.vc = reinterpret_cast<half_t *>(d.desc->v_cache[z]) + d.cache_offset;
    int pos = d.desc->pos[z];
    if (pos > a.max_pos - 1) pos = a.max_pos - 1;
    a.pos_host = pos < 0 ? 0 : pos;
}

template <bool DEV>
__device__ __forceinline__ AdArgs ad_for_sequence(const AdArgs &common, const AdBatch &b, const AdBatchDev &d, int z) {
    AdArgs a = common;
    a.q = b.qkv + (size_t)z * b.ldq;
    a.out = b.out + (size_t)z * b.ldo;
    if (DEV) ad_sequence_caches(b, d, z, a, 0);
    else ad_sequence_caches(b, d, z, a);
    a.pos_dev = nullptr;
    if (a.ws_acc) {
        a.ws_acc += (size_t)z * b.ws_floats;
        a.ws_ml += (size_t)z * b.ws_floats;
    }
    return a;
}

// every position below 512: the single-span form (dim-split workgroups, direct result)
template <int HD, int G, int DSN, bool DEV>
__global__ __launch_bounds__(AD_THREADS) void attn_decode_batch_kernel(const AdArgs common, const AdBatch b, const AdBatchDev d) {
    __shared__ float sc[G * AD_LS];
    __shared__ __attribute__((aligned(16))) half_t qs[G * HD];
    __shared__ __attribute__((aligned(16))) half_t knew[HD];
    __shared__ __attribute__((aligned(16))) half_t vnew[HD];
    __shared__ float s_m[G], s_l[G];
    __shared__ int s_last;
    AdArgs a = ad_for_sequence<DEV>(common, b, d, blockIdx.z);
    if (a.pos_host > AD_LS - 1) a.pos_host = AD_LS - 1; // this form serves one span; the host picks it below AD_LS only
    const int y = blockIdx.y;
    attn_decode_body<HD, G, true, HD / DSN, AD_LS>(a, sc, qs, knew, vnew, s_m, s_l, &s_last, a.pos_host, 1, 0,
                                                   y * (HD / DSN), y == 0);
}

template <int HD, int G, bool DEV>
__global__ __launch_bounds__(AD_SPAN_THREADS, 4) void attn_span_batch_kernel(const AdArgs common, const AdBatch b, const AdBatchDev d) {
    const AdArgs a = ad_for_sequence<DEV>(common, b, d, blockIdx.z);
    const int span = ad_long_span(a.pos_host + 1, a.span_target);
    const int n_active = (a.pos_host + span) / span;
    const int y = blockIdx.y;
    if (y >= n_active) return;
    if (y == n_active - 1) attn_span_wave<HD, G, true>(a, a.pos_host, y, blockIdx.x, span);
    else attn_span_wave<HD, G, false>(a, a.pos_host, y, blockIdx.x, span);
}

template <int HD, int G, bool DEV>
__global__ __launch_bounds__(AD_MERGE_THREADS) void attn_merge_batch_kernel(const AdArgs common, const AdBatch b, const AdBatchDev d) {
    attn_merge_body<HD, G>(ad_for_sequence<DEV>(common, b, d, blockIdx.y), blockIdx.x);
}

// long_form: < 0 decides from the host's positions in b; with a descriptor in device memory the caller decides
// (0: every position below AD_LS, 1: the span + merge form) and the span grid covers any position below max_pos.
template <int HD, int G>
static int launch_decode_batch(AdArgs a, const AdBatch &b, const AdBatchDev &d, int long_form, int B, void *ws, hipStream_t s) {
    constexpr int DSN = HD >= 128 ? 4 : 1;
    const int Hq = a.n_kv_heads * G;
    const bool dev = d.desc != nullptr;
    if (long_form < 0) {
        int max_pos_used = 0;
        for (int z = 0; z < B; ++z) max_pos_used = b.pos[z] > max_pos_used ? b.pos[z] : max_pos_used;
        long_form = max_pos_used < AD_LS ? 0 : 1;
    }
    if (!long_form) {
        a.ws_acc = nullptr;
        if (dev) attn_decode_batch_kernel<HD, G, DSN, true><<<dim3(a.n_kv_heads, DSN, B), dim3(AD_THREADS), 0, s>>>(a, b, d);
        else attn_decode_batch_kernel<HD, G, DSN, false><<<dim3(a.n_kv_heads, DSN, B), dim3(AD_THREADS), 0, s>>>(a, b, d);
        LLM_LAUNCH_CHECK("attn_decode_batch_kernel");
        return LLM_OK;
    }
    a.ws_acc = (float *)ws;
    a.ws_ml = a.ws_acc + (size_t)Hq * AD_MAX_SPLITS * HD;
    int gy = 0;
    a.pos_dev = nullptr;
    a.pos_host = 0;
    int rc = ad_long_setup(a, &gy);
    if (rc != LLM_OK) return rc;
    if (dev) {
        gy = a.splits; // any position below max_pos
        attn_span_batch_kernel<HD, G, true><<<dim3(a.n_kv_heads, gy, B), dim3(AD_SPAN_THREADS), 0, s>>>(a, b, d);
        LLM_LAUNCH_CHECK("attn_span_batch_kernel");
        attn_merge_batch_kernel<HD, G, true><<<dim3(Hq, B), dim3(AD_MERGE_THREADS), 0, s>>>(a, b, d);
        LLM_LAUNCH_CHECK("attn_merge_batch_kernel");
        return LLM_OK;
    }
    gy = 1;
    for (int z = 0; z < B; ++z) { // the sequence with the most spans sizes the grid (not always the longest one)
        const int n = ad_long_spans(b.pos[z] + 1, a.span_target);
        gy = n > gy ? n : gy;
    }
    attn_span_batch_kernel<HD, G, false><<<dim3(a.n_kv_heads, gy, B), dim3(AD_SPAN_THREADS), 0, s>>>(a, b, d);
    LLM_LAUNCH_CHECK("attn_span_batch_kernel");
    attn_merge_batch_kernel<HD, G, false><<<dim3(Hq, B), dim3(AD_MERGE_THREADS), 0, s>>>(a, b, d);
    LLM_LAUNCH_CHECK("attn_merge_batch_kernel");
    return LLM_OK;
}

static int dispatch_decode_long(AdArgs a, int n_heads, int head_dim, void *ws, hipStream_t s) {
    const int G = n_heads / a.n_kv_heads;
#define AD_CASE(HD_, G_) \
    if (head_dim == HD_ && G == G_) return launch_decode_long<HD_, G_>(a, ws, s);
    AD_CASE(128, 4)
    AD_CASE(128, 8)
    AD_CASE(128, 1)
    AD_CASE(64, 4)
    AD_CASE(64, 1)
    AD_CASE(32, 4)
    AD_CASE(32, 1)
#undef AD_CASE
    llm_set_error("llm_attn_decode: head_dim=%d with group size %d is not built", head_dim, G);
    return LLM_ERR_INVALID;
}

extern "C" {

// Layout: acc [Hq][AD_MAX_SPLITS][hd] floats, (m,l) [Hq][AD_MAX_SPLITS][2]
// floats, then one int counter per KV head (<= Hq of them).  The counters must
// be zero before the first launch (llm_fill_zero the workspace once); every
// launch leaves them zero.
size_t llm_attn_decode_workspace_bytes(int n_heads, int head_dim) {
    return sizeof(float) * (size_t)n_heads * AD_MAX_SPLITS * (head_dim + 2) + sizeof(int) * (size_t)n_heads;
}

// what llm_attn_decode and llm_attn_decode_noalloc require of their arguments, checked before either launches anything
static int attn_decode_check(const void *q, const void *kc, const void *vc, const void *out, int ctx_host,
                             const int32_t *ctx_dev, int n_heads, int n_kv_heads, int head_dim, int max_pos) {
    LLM_REQUIRE(q && kc && vc && out, "llm_attn_decode: null pointer");
    LLM_REQUIRE(n_kv_heads > 0 && n_heads > 0 && n_heads % n_kv_heads == 0, "llm_attn_decode: heads %d/%d", n_heads, n_kv_heads);
    LLM_REQUIRE(max_pos > 0 && max_pos % 64 == 0, "llm_attn_decode: max_pos=%d must be a multiple of 64", max_pos);
    LLM_REQUIRE((max_pos + AD_LS - 1) / AD_LS <= AD_MAX_SPLITS, "llm_attn_decode: max_pos=%d exceeds %d", max_pos, AD_MAX_SPLITS * AD_LS);
    LLM_REQUIRE(ctx_dev || (ctx_host >= 1 && ctx_host <= max_pos), "llm_attn_decode: ctx=%d of %d", ctx_host, max_pos);
    LLM_REQUIRE(aligned16(q) && aligned16(kc) && aligned16(vc), "llm_attn_decode: pointers must be 16-byte aligned");
    const int G = n_heads / n_kv_heads;
    const bool built = (head_dim == 128 && (G == 1 || G == 4 || G == 8)) || ((head_dim == 64 || head_dim == 32) && (G == 1 || G == 4));
    LLM_REQUIRE(built, "llm_attn_decode: head_dim=%d with group size %d is not built", head_dim, G);
    return LLM_OK;
}

int llm_attn_decode(const uint16_t *q, const uint16_t *kc, const uint16_t *vc, uint16_t *out, int ctx_host,
                    const int32_t *ctx_dev, int n_heads, int n_kv_heads, int head_dim, int max_pos, void *workspace,
                    llm_stream_t stream) {
    LLM_REQUIRE(workspace, "llm_attn_decode: null workspace");
    int rc = attn_decode_check(q, kc, vc, out, ctx_host, ctx_dev, n_heads, n_kv_heads, head_dim, max_pos);
    if (rc != LLM_OK) return rc;
    AdArgs a = {};
    a.q = (const half_t *)q;
    a.kc = (half_t *)kc;
    a.vc = (half_t *)vc;
    a.out = (half_t *)out;
    a.pos_host = ctx_host - 1;
    a.pos_dev = ctx_dev;
    a.n_kv_heads = n_kv_heads;
    a.max_pos = max_pos;
    return dispatch_decode<false>(a, n_heads, head_dim, workspace, (hipStream_t)stream);
}

// ---- the same operation for callers that cannot allocate -------------------------------------
// The partial results (acc, m, l per span) and the per-KV-head counters live in a file-scope device
// array sized for 32 query heads of 128 dims (LLaMA3-8B): 4 259 968 bytes on every GPU the library
// runs on, held until the process ends.  The array's name is only a host-side handle; the device
// address is fetched per device with hipGetSymbolAddress and that pointer is what kernels get.
#define AD_STATIC_MAX_HEADS 32
#define AD_STATIC_MAX_HEAD_DIM 128
#define AD_STATIC_BYTES \
    (sizeof(float) * AD_STATIC_MAX_HEADS * AD_MAX_SPLITS * (AD_STATIC_MAX_HEAD_DIM + 2) + sizeof(int) * AD_STATIC_MAX_HEADS)
static __device__ __align__(256) unsigned char scratch[AD_STATIC_BYTES];

#define AD_MAX_DEVICES 64
static void *g_scratch_ptr[AD_MAX_DEVICES];
static std::mutex g_scratch_mutex;

// Device address of this device's copy of the array (the current device must be `device`).
static int scratch_for_device(int device, void **ptr) {
    LLM_REQUIRE(device >= 0 && device < AD_MAX_DEVICES, "llm_attn_decode_noalloc: device %d out of range", device);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void *p = nullptr;
        LLM_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        LLM_REQUIRE(p != nullptr, "llm_attn_decode_noalloc: no device address for the scratch array");
        g_scratch_ptr[device] = p;
    }
    *ptr = g_scratch_ptr[device];
    return LLM_OK;
}

// Called by llm_init with the selected device current.
int attn_decode_static_setup(int device) {
    void *p;
    return scratch_for_device(device, &p);
}

size_t llm_attn_decode_noalloc_max_bytes(void) { return AD_STATIC_BYTES; }

int llm_attn_decode_noalloc(const uint16_t *q, const uint16_t *kc, const uint16_t *vc, uint16_t *out, int ctx_host,
                            const int32_t *ctx_dev, int n_heads, int n_kv_heads, int head_dim, int max_pos,
                            llm_stream_t stream) {
    LLM_REQUIRE(n_heads > 0 && head_dim > 0, "llm_attn_decode_noalloc: heads %d, head_dim %d", n_heads, head_dim);
    const size_t need = llm_attn_decode_workspace_bytes(n_heads, head_dim);
    LLM_REQUIRE(n_heads <= AD_STATIC_MAX_HEADS && head_dim <= AD_STATIC_MAX_HEAD_DIM && need <= AD_STATIC_BYTES,
                "llm_attn_decode_noalloc: %d heads of %d dims need %zu scratch bytes; the built-in scratch holds %zu "
                "(at most %d heads of at most %d dims): use llm_attn_decode with a workspace",
                n_heads, head_dim, need, (size_t)AD_STATIC_BYTES, AD_STATIC_MAX_HEADS, AD_STATIC_MAX_HEAD_DIM);
    // every argument is checked before the first launch: an invalid call enqueues nothing
    int rc = attn_decode_check(q, kc, vc, out, ctx_host, ctx_dev, n_heads, n_kv_heads, head_dim, max_pos);
    if (rc != LLM_OK) return rc;
    int device = 0;
    LLM_HIP_CHECK(hipGetDevice(&device));
    void *ws = nullptr;
    rc = scratch_for_device(device, &ws);
    if (rc != LLM_OK) return rc;
    // The array keeps what the last call left, and the counters sit behind the partial results at an
    // offset that depends on (n_heads, head_dim): after a call with another shape that spot holds
    // floats.  Clear this shape's counters with a fill kernel (safe under graph capture).
    char *counters = (char *)ws + sizeof(float) * (size_t)n_heads * AD_MAX_SPLITS * (head_dim + 2);
    rc = llm_fill_zero(counters, sizeof(int) * (size_t)n_heads, stream);
    if (rc != LLM_OK) return rc;
    return llm_attn_decode(q, kc, vc, out, ctx_host, ctx_dev, n_heads, n_kv_heads, head_dim, max_pos, ws, stream);
}

int llm_attn_decode_rope(const uint16_t *qkv, uint16_t *kc, uint16_t *vc, uint16_t *out, int pos_host,
                         const int32_t *pos_dev, const float *table, int n_heads, int n_kv_heads, int head_dim,
                         int max_pos, void *workspace, llm_stream_t stream) {
    LLM_REQUIRE(qkv && kc && vc && out && table && workspace, "llm_attn_decode_rope: null pointer");
    LLM_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "llm_attn_decode_rope: heads %d/%d", n_heads, n_kv_heads);
    LLM_REQUIRE(max_pos > 0 && max_pos % 64 == 0, "llm_attn_decode_rope: max_pos=%d must be a multiple of 64", max_pos);
    LLM_REQUIRE(pos_dev || (pos_host >= 0 && pos_host < max_pos), "llm_attn_decode_rope: position %d of %d", pos_host,
                max_pos);
    LLM_REQUIRE(aligned16(qkv) && aligned16(kc) && aligned16(vc), "llm_attn_decode_rope: pointers must be 16-byte aligned");
    AdArgs a = {};
    a.q = (const half_t *)qkv;
    a.kc = (half_t *)kc;
    a.vc = (half_t *)vc;
    a.out = (half_t *)out;
    a.table = table;
    a.pos_host = pos_host;
    a.pos_dev = pos_dev;
    a.n_kv_heads = n_kv_heads;
    a.max_pos = max_pos;
    return dispatch_decode<true>(a, n_heads, head_dim, workspace, (hipStream_t)stream);
}

int llm_attn_decode_rope_oproj(const uint16_t *qkv, uint16_t *kc, uint16_t *vc, uint16_t *attn_out, uint16_t *attn_out_next,
                               int pos_host, const int32_t *pos_dev, const float *table, int n_heads, int n_kv_heads,
                               int head_dim, int max_pos, const uint16_t *w, const uint16_t *residual, uint16_t *out, int N,
                               int32_t *timeouts_dev, int spin_limit, llm_stream_t stream) {
    LLM_REQUIRE(qkv && kc && vc && attn_out && attn_out_next && table && w && out && timeouts_dev,
                "llm_attn_decode_rope_oproj: null pointer");
    LLM_REQUIRE(attn_out != attn_out_next, "llm_attn_decode_rope_oproj: a launch cannot refill its own buffer");
    LLM_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "llm_attn_decode_rope_oproj: heads %d/%d", n_heads, n_kv_heads);
    LLM_REQUIRE(max_pos > 0 && max_pos % 64 == 0, "llm_attn_decode_rope_oproj: max_pos=%d must be a multiple of 64", max_pos);
    LLM_REQUIRE(pos_dev || (pos_host >= 0 && pos_host < max_pos && pos_host < AD_LS),
                "llm_attn_decode_rope_oproj: position %d (must be below %d and below max_pos %d)", pos_host, AD_LS, max_pos);
    const int K = n_heads * head_dim;
    LLM_REQUIRE(N > 0 && K % 8 == 0 && K <= 512 * AO_KSTEPS, "llm_attn_decode_rope_oproj: N=%d K=%d (K <= %d)", N, K,
                512 * AO_KSTEPS);
    LLM_REQUIRE(aligned16(qkv) && aligned16(kc) && aligned16(vc) && aligned16(attn_out) && aligned16(attn_out_next) &&
                    aligned16(w),
                "llm_attn_decode_rope_oproj: pointers must be 16-byte aligned");
    AdArgs a = {};
    a.q = (const half_t *)qkv;
    a.kc = (half_t *)kc;
    a.vc = (half_t *)vc;
    a.out = (half_t *)attn_out;
    a.table = table;
    a.pos_host = pos_host;
    a.pos_dev = pos_dev;
    a.n_kv_heads = n_kv_heads;
    a.max_pos = max_pos;
    AoArgs o = {};
    o.w = (const half_t *)w;
    o.res = (const half_t *)residual;
    o.out = (half_t *)out;
    o.next = attn_out_next;
    o.N = N;
    o.K = K;
    o.timeouts = timeouts_dev;
    o.spin_limit = spin_limit >= 0 ? spin_limit : AO_SPIN_LIMIT;
    hipStream_t s = (hipStream_t)stream;
    const int G = n_heads / n_kv_heads;
#define AO_CASE(HD_, G_) \
    if (head_dim == HD_ && G == G_) return launch_attn_oproj<HD_, G_>(a, o, s);
    AO_CASE(128, 4)
    AO_CASE(128, 8)
    AO_CASE(128, 1)
    AO_CASE(64, 4)
    AO_CASE(64, 1)
    AO_CASE(32, 4)
    AO_CASE(32, 1)
#undef AO_CASE
    llm_set_error("llm_attn_decode_rope_oproj: head_dim=%d with group size %d is not built", head_dim, G);
    return LLM_ERR_INVALID;
}

// 1 when llm_attn_decode_rope_oproj covers these shapes on the current device, else 0.
int llm_attn_oproj_supported(int n_heads, int n_kv_heads, int head_dim, int N) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads) return 0;
    const int G = n_heads / n_kv_heads, K = n_heads * head_dim;
    if (!((head_dim == 128 && (G == 1 || G == 4 || G == 8)) || ((head_dim == 64 || head_dim == 32) && (G == 1 || G == 4)))) return 0;
    if (K % 8 || K > 512 * AO_KSTEPS || (size_t)K * sizeof(half_t) > sizeof(float) * G * AD_LS || N <= 0) return 0;
    int cus = 0;
    if (llm_cu_count_cached(&cus) != LLM_OK) return 0;
    const int n_attn = n_kv_heads * (head_dim >= 128 ? 4 : 1);
    if (cus <= n_attn) return 0;
    int owg = (N + AO_WAVES - 1) / AO_WAVES;
    if (owg > cus - n_attn) owg = cus - n_attn;
    return (N + owg * AO_WAVES - 1) / (owg * AO_WAVES) <= AO_ROWS;
}

// Fills n fp16 slots with the "not written yet" pattern of llm_attn_decode_rope_oproj (a fill kernel:
// safe under graph capture).
__global__ void ao_fill_empty_kernel(uint16_t *p, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = AO_EMPTY;
}
int llm_attn_oproj_buffer_init(uint16_t *buf, int n, llm_stream_t stream) {
    LLM_REQUIRE(buf && n > 0, "llm_attn_oproj_buffer_init: buf/n");
    ao_fill_empty_kernel<<<dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream>>>(buf, n);
    LLM_LAUNCH_CHECK("ao_fill_empty_kernel");
    return LLM_OK;
}

int llm_attn_decode_rope_long(const uint16_t *qkv, uint16_t *kc, uint16_t *vc, uint16_t *out, int pos_host,
                         const int32_t *pos_dev, const float *table, int n_heads, int n_kv_heads, int head_dim,
                         int max_pos, void *workspace, llm_stream_t stream) {
    LLM_REQUIRE(qkv && kc && vc && out && table && workspace, "llm_attn_decode_rope_long: null pointer");
    LLM_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "llm_attn_decode_rope_long: heads %d/%d", n_heads, n_kv_heads);
    LLM_REQUIRE(max_pos > 0 && max_pos % 64 == 0, "llm_attn_decode_rope_long: max_pos=%d must be a multiple of 64", max_pos);
    LLM_REQUIRE(pos_dev || (pos_host >= 0 && pos_host < max_pos), "llm_attn_decode_rope_long: position %d of %d", pos_host,
                max_pos);
    LLM_REQUIRE(aligned16(qkv) && aligned16(kc) && aligned16(vc), "llm_attn_decode_rope_long: pointers must be 16-byte aligned");
    AdArgs a = {};
    a.q = (const half_t *)qkv;
    a.kc = (half_t *)kc;
    a.vc = (half_t *)vc;
    a.out = (half_t *)out;
    a.table = table;
    a.pos_host = pos_host;
    a.pos_dev = pos_dev;
    a.n_kv_heads = n_kv_heads;
    a.max_pos = max_pos;
    return dispatch_decode_long(a, n_heads, head_dim, workspace, (hipStream_t)stream);
}

// 1 when llm_attn_decode_rope_long_oproj covers these shapes on the current device, else 0.
int llm_attn_long_oproj_supported(int n_heads, int n_kv_heads, int head_dim, int N) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads) return 0;
    const int G = n_heads / n_kv_heads, K = n_heads * head_dim;
    if (!((head_dim == 128 && (G == 1 || G == 4 || G == 8)) || ((head_dim == 64 || head_dim == 32) && (G == 1 || G == 4)))) return 0;
    if (K % 8 || K > 512 * AO_KSTEPS || N <= 0) return 0;
    int cus = 0, owg = 0, rows = 0;
    if (llm_cu_count_cached(&cus) != LLM_OK) return 0;
    return ao_partition(N, n_heads, cus, &owg, &rows) ? 1 : 0;
}

int llm_attn_decode_rope_long_oproj(const uint16_t *qkv, uint16_t *kc, uint16_t *vc, uint16_t *attn_out,
                                    uint16_t *attn_out_next, int pos_host, const int32_t *pos_dev, const float *table,
                                    int n_heads, int n_kv_heads, int head_dim, int max_pos, void *workspace,
                                    const uint16_t *w, const uint16_t *residual, uint16_t *out, int N,
                                    int32_t *timeouts_dev, int spin_limit, llm_stream_t stream) {
    LLM_REQUIRE(qkv && kc && vc && attn_out && attn_out_next && table && workspace && w && out && timeouts_dev,
                "llm_attn_decode_rope_long_oproj: null pointer");
    LLM_REQUIRE(attn_out != attn_out_next, "llm_attn_decode_rope_long_oproj: a launch cannot refill its own buffer");
    LLM_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "llm_attn_decode_rope_long_oproj: heads %d/%d", n_heads, n_kv_heads);
    LLM_REQUIRE(max_pos > 0 && max_pos % 64 == 0, "llm_attn_decode_rope_long_oproj: max_pos=%d must be a multiple of 64", max_pos);
    LLM_REQUIRE(pos_dev || (pos_host >= 0 && pos_host < max_pos), "llm_attn_decode_rope_long_oproj: position %d of %d", pos_host,
                max_pos);
    const int K = n_heads * head_dim;
    LLM_REQUIRE(N > 0 && K % 8 == 0 && K <= 512 * AO_KSTEPS, "llm_attn_decode_rope_long_oproj: N=%d K=%d (K <= %d)", N, K,
                512 * AO_KSTEPS);
    LLM_REQUIRE(aligned16(qkv) && aligned16(kc) && aligned16(vc) && aligned16(attn_out) && aligned16(attn_out_next) &&
                    aligned16(w),
                "llm_attn_decode_rope_long_oproj: pointers must be 16-byte aligned");
    AdArgs a = {};
    a.q = (const half_t *)qkv;
    a.kc = (half_t *)kc;
    a.vc = (half_t *)vc;
    a.out = (half_t *)attn_out;
    a.table = table;
    a.pos_host = pos_host;
    a.pos_dev = pos_dev;
    a.n_kv_heads = n_kv_heads;
    a.max_pos = max_pos;
    AoArgs o = {};
    o.w = (const half_t *)w;
    o.res = (const half_t *)residual;
    o.out = (half_t *)out;
    o.next = attn_out_next;
    o.N = N;
    o.K = K;
    o.timeouts = timeouts_dev;
    o.spin_limit = spin_limit >= 0 ? spin_limit : AO_SPIN_LIMIT;
    hipStream_t s = (hipStream_t)stream;
    const int G = n_heads / n_kv_heads;
#define AO_CASE(HD_, G_) \
    if (head_dim == HD_ && G == G_) return launch_long_oproj<HD_, G_>(a, o, workspace, s);
    AO_CASE(128, 4)
    AO_CASE(128, 8)
    AO_CASE(128, 1)
    AO_CASE(64, 4)
    AO_CASE(64, 1)
    AO_CASE(32, 4)
    AO_CASE(32, 1)
#undef AO_CASE
    llm_set_error("llm_attn_decode_rope_long_oproj: head_dim=%d with group size %d is not built", head_dim, G);
    return LLM_ERR_INVALID;
}

int llm_attn_decode_rope_batch(const uint16_t *qkv, int ldq, uint16_t *const *k_caches, uint16_t *const *v_caches,
                               const int *positions, int batch, uint16_t *out, int ldo, const float *table,
                               int n_heads, int n_kv_heads, int head_dim, int max_pos, void *workspace,
                               llm_stream_t stream) {
    LLM_REQUIRE(qkv && k_caches && v_caches && positions && out && table && workspace, "llm_attn_decode_rope_batch: null pointer");
    LLM_REQUIRE(batch >= 1 && batch <= AD_MAX_BATCH, "llm_attn_decode_rope_batch: batch=%d (1..%d)", batch, AD_MAX_BATCH);
    LLM_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "llm_attn_decode_rope_batch: heads %d/%d", n_heads, n_kv_heads);
    LLM_REQUIRE(max_pos > 0 && max_pos % 64 == 0, "llm_attn_decode_rope_batch: max_pos=%d must be a multiple of 64", max_pos);
    LLM_REQUIRE(ldq % 8 == 0 && ldq >= (n_heads + 2 * n_kv_heads) * head_dim && ldo >= n_heads * head_dim,
                "llm_attn_decode_rope_batch: ldq=%d ldo=%d", ldq, ldo);
    LLM_REQUIRE(aligned16(qkv), "llm_attn_decode_rope_batch: qkv must be 16-byte aligned");
    AdBatch b = {};
    b.qkv = (const half_t *)qkv;
    b.ldq = ldq;
    b.out = (half_t *)out;
    b.ldo = ldo;
    b.ws_floats = llm_attn_decode_workspace_bytes(n_heads, head_dim) / sizeof(float);
    for (int z = 0; z < batch; ++z) {
        LLM_REQUIRE(k_caches[z] && v_caches[z] && aligned16(k_caches[z]) && aligned16(v_caches[z]),
                    "llm_attn_decode_rope_batch: cache %d", z);
        LLM_REQUIRE(positions[z] >= 0 && positions[z] < max_pos, "llm_attn_decode_rope_batch: position %d of %d",
                    positions[z], max_pos);
        b.kc[z] = (half_t *)k_caches[z];
        b.vc[z] = (half_t *)v_caches[z];
        b.pos[z] = positions[z];
    }
    AdArgs a = {};
    a.table = table;
    a.n_kv_heads = n_kv_heads;
    a.max_pos = max_pos;
    const int G = n_heads / n_kv_heads;
    hipStream_t s = (hipStream_t)stream;
    const AdBatchDev d = {nullptr, 0};
#define AD_CASE(HD_, G_) \
    if (head_dim == HD_ && G == G_) return launch_decode_batch<HD_, G_>(a, b, d, -1, batch, workspace, s);
    AD_CASE(128, 4)
    AD_CASE(128, 8)
    AD_CASE(128, 1)
    AD_CASE(64, 4)
    AD_CASE(64, 1)
    AD_CASE(32, 4)
    AD_CASE(32, 1)
#undef AD_CASE
    llm_set_error("llm_attn_decode_rope_batch: head_dim=%d with group size %d is not built", head_dim, G);
    return LLM_ERR_INVALID;
}

int llm_attn_decode_rope_batch_dev(const uint16_t *qkv, int ldq, const llm_batch_desc *desc_dev, size_t cache_offset, int batch,
                                   int long_form, uint16_t *out, int ldo, const float *table, int n_heads, int n_kv_heads,
                                   int head_dim, int max_pos, void *workspace, llm_stream_t stream) {
    LLM_REQUIRE(qkv && desc_dev && out && table && workspace, "llm_attn_decode_rope_batch_dev: null pointer");
    LLM_REQUIRE(batch >= 1 && batch <= AD_MAX_BATCH && LLM_MAX_BATCH == AD_MAX_BATCH, "llm_attn_decode_rope_batch_dev: batch=%d (1..%d)",
                batch, AD_MAX_BATCH);
    LLM_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "llm_attn_decode_rope_batch_dev: heads %d/%d", n_heads, n_kv_heads);
    LLM_REQUIRE(max_pos > 0 && max_pos % 64 == 0, "llm_attn_decode_rope_batch_dev: max_pos=%d must be a multiple of 64", max_pos);
    LLM_REQUIRE(ldq % 8 == 0 && ldq >= (n_heads + 2 * n_kv_heads) * head_dim && ldo >= n_heads * head_dim,
                "llm_attn_decode_rope_batch_dev: ldq=%d ldo=%d", ldq, ldo);
    LLM_REQUIRE(aligned16(qkv) && cache_offset % 8 == 0, "llm_attn_decode_rope_batch_dev: qkv and the cache offset must be 16-byte aligned");
    LLM_REQUIRE(long_form == 0 || long_form == 1, "llm_attn_decode_rope_batch_dev: long_form is 0 or 1");
    AdBatch b = {};
    b.qkv = (const half_t *)qkv;
    b.ldq = ldq;
    b.out = (half_t *)out;
    b.ldo = ldo;
    b.ws_floats = llm_attn_decode_workspace_bytes(n_heads, head_dim) / sizeof(float);
    const AdBatchDev d = {desc_dev, cache_offset};
    AdArgs a = {};
    a.table = table;
    a.n_kv_heads = n_kv_heads;
    a.max_pos = max_pos;
    const int G = n_heads / n_kv_heads;
    hipStream_t s = (hipStream_t)stream;
#define AD_CASE(HD_, G_) \
    if (head_dim == HD_ && G == G_) return launch_decode_batch<HD_, G_>(a, b, d, long_form, batch, workspace, s);
    AD_CASE(128, 4)
    AD_CASE(128, 8)
    AD_CASE(128, 1)
    AD_CASE(64, 4)
    AD_CASE(64, 1)
    AD_CASE(32, 4)
    AD_CASE(32, 1)
#undef AD_CASE
    llm_set_error("llm_attn_decode_rope_batch_dev: head_dim=%d with group size %d is not built", head_dim, G);
    return LLM_ERR_INVALID;
}

} // extern "C"
