// Candidate selection for the reference's sampler on the device (src/inference/inference.cu:1043-1161):
// the softmax denominator exactly as the host loop accumulates it, and the k entries that the descending
// qsort of the whole vocabulary would put first, so that the host draws from k pairs instead of exponentiating,
// normalising and sorting 128256 logits per token.
//
// Everything that decides a draw is reproduced bit for bit:
//   * exp(logit / temperature) comes from a 65536-entry table the host fills with its own expf (one entry per
//     fp16 bit pattern), not from the device's exp;
//   * the denominator is the float32 running sum in index order (seqsum.hpp);
//   * probabilities are table[logit] / denominator with the correctly rounded float32 division;
//   * order is (probability descending, index ascending): what a stable sort of the reference's array by
//     _compare_desc leaves.  Distinct logits can round to the same probability, so the cut is made on the
//     probability, not on the logit: everything above the k-th largest logit's probability, then the
//     lowest-indexed entries equal to it.
// One launch of ceil(vocab / 2048) workgroups of 256 threads that meet at grid-wide barriers (all of them are
// resident at once: at most SC_MAX_WG, far fewer than the device has compute units).  A thread owns 8
// consecutive entries, kept in registers throughout; a wavefront owns the 512 entries of its lanes, the unit
// of the running sum's exponent guess.
#include "common.hpp"
#include "seqsum.hpp"

#define SC_WG 256
#define SC_WAVES (SC_WG / 64)
#define SC_PER_WG (SC_WG * 8)
#define SC_MAX_WG 128
#define SC_MAX_SEG (SC_MAX_WG * SC_WAVES)
#define SC_SPIN_LIMIT (1 << 20)
#define SC_LANE_WORDS64 6 // 8-byte words per thread behind the control block

namespace {

// 32-bit words of the control block that follows the head of the output; zeroed before every launch
enum {
    C_BARRIER = 0,  // 5 arrival counters
    C_TIMEOUT = 5,  // a barrier gave up waiting
    C_DENOM = 6,    // bits of the denominator
    C_ONE_BY_ONE = 7,
    C_BAD = 8,      // a value the selection cannot handle was seen
    C_HIST1 = 16,   // entries by upper byte of the order key
    C_HIST2 = C_HIST1 + 256,
    C_WG_GT = C_HIST2 + 256, // per workgroup: entries above / equal to the cut
    C_WG_EQ = C_WG_GT + SC_MAX_WG,
    C_SEG_SUM = C_WG_EQ + SC_MAX_WG, // per wavefront range: approximate sum, composed run, exponent guess
    C_SEG_A0 = C_SEG_SUM + SC_MAX_SEG,
    C_SEG_A1 = C_SEG_A0 + SC_MAX_SEG,
    C_SEG_ES = C_SEG_A1 + SC_MAX_SEG,
    C_SEG_BASE = C_SEG_ES + SC_MAX_SEG, // exponent the per-thread runs were computed for (and the next one)
    C_WORDS = C_SEG_BASE + SC_MAX_SEG
};

__host__ __device__ inline size_t sc_head_bytes(int k) { return (16 + 8 * (size_t)k + 15) & ~(size_t)15; }
__host__ __device__ inline int sc_workgroups(int vocab) { return (vocab + SC_PER_WG - 1) / SC_PER_WG; }

__device__ __forceinline__ uint32_t ld_agent(const uint32_t *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void st_agent(uint32_t *p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent64(unsigned long long *p, unsigned long long v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// What the walking wavefront needs of one range when it has to go through it lane by lane: per lane the two
// runs and the 8 values, fetched with independent loads so that one memory latency covers them all.
struct ScRange {
    unsigned long long w[6];
};
__device__ __forceinline__ void sc_fetch_range(ScRange &r, const unsigned long long *lane_data, int range, int lane) {
    const unsigned long long *theirs = lane_data + (size_t)(range * 64 + lane) * 6;
#pragma unroll
    for (int i = 0; i < 6; ++i) r.w[i] = __hip_atomic_load(theirs + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Every workgroup of the grid arrives before any leaves.  Data that crosses workgroups goes through
// device-scope stores and loads (st_agent / ld_agent / atomics), which bypass the caches that are private to a
// compute unit or to a die, so no cache write-back or invalidation is needed here: a thread waits until its
// own stores have been acknowledged, the workgroup meets, then one thread announces the arrival.  The wait is
// bounded: a barrier that gives up raises C_TIMEOUT, which invalidates the result.
__device__ __forceinline__ void grid_barrier(uint32_t *ctrl, int which, int nwg) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        atomicAdd(&ctrl[C_BARRIER + which], 1u);
        int spins = 0;
        while (ld_agent(&ctrl[C_BARRIER + which]) < (uint32_t)nwg) {
            __builtin_amdgcn_s_sleep(4);
            if (++spins > SC_SPIN_LIMIT) {
                atomicOr(&ctrl[C_TIMEOUT], 1u);
                break;
            }
        }
    }
    __syncthreads();
}

// Exclusive prefix over the block in thread order and the block total (both for every thread).
template <typename T> __device__ __forceinline__ T block_exclusive(T v, T *wave_tot, T &total) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    T inc = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        T o = __shfl_up(inc, d);
        if (lane >= d) inc += o;
    }
    __syncthreads(); // wave_tot may still be read from a previous call
    if (lane == 63) wave_tot[w] = inc;
    __syncthreads();
    T before = 0, all = 0;
#pragma unroll
    for (int i = 0; i < SC_WAVES; ++i) {
        T t = wave_tot[i];
        if (i < w) before += t;
        all += t;
    }
    total = all;
    return before + inc - v;
}

__device__ __forceinline__ uint16_t key_to_bits(uint32_t key) {
    return key >= 0x8000u ? (uint16_t)(key - 0x8000u) : (uint16_t)(0x8000u | (0x7fffu - key));
}

// Largest byte value b such that at least `want` counted entries have a byte >= b; above = entries with a
// larger byte.  hist[256] in LDS, complete and visible; every thread returns the same answer.
__device__ __forceinline__ int pick_bin(const uint32_t *hist, uint32_t want, uint32_t &above) {
    uint32_t acc = 0;
    int b = 255;
    for (; b > 0; --b) {
        const uint32_t h = hist[b];
        if (acc + h >= want) break;
        acc += h;
    }
    above = acc;
    return b;
}

// Adds this thread's 8 bytes (bin[u], counted where take[u]) to an LDS histogram, equal neighbours at once.
__device__ __forceinline__ void hist_add8(uint32_t *hist, const uint32_t (&bin)[8], const bool (&take)[8]) {
    uint32_t run_bin = 0xffffffffu, run = 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        if (!take[u]) continue;
        if (bin[u] != run_bin) {
            if (run) atomicAdd(&hist[run_bin], run);
            run_bin = bin[u];
            run = 0;
        }
        ++run;
    }
    if (run) atomicAdd(&hist[run_bin], run);
}

// One run per lane (m, lanes [from, cnt)), all computed for biased exponent es: applies to s the longest
// prefix of them, in lane order, that is usable and keeps s inside that binade, and returns the first lane
// that was not applied (cnt when all were).  The prefixes are composed by a scan and tested in all lanes at
// once, so the cost does not grow with the number of runs.  s, from, cnt, es: the same in every lane.
__device__ __forceinline__ int sc_apply_prefix(uint32_t &s, SeqMap m, bool usable, int from, int cnt, int es, int lane) {
    if (es < 1 || es > 253 || (int)(s >> 23) != es) return from;
    const bool mine = lane >= from && lane < cnt;
    SeqMap pm = {mine ? m.a0 : 0u, mine ? m.a1 : 0u};
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        SeqMap earlier;
        earlier.a0 = __shfl_up(pm.a0, d);
        earlier.a1 = __shfl_up(pm.a1, d);
        if (lane >= d) pm = seqmap_compose(earlier, pm);
    }
    const uint32_t S = (s & 0x7fffffu) | 0x800000u;
    const uint32_t S2 = S + ((S & 1u) ? pm.a1 : pm.a0);
    // an unusable run or a sum that leaves the binade stops the prefix; increments only grow along the lanes
    const unsigned long long stop = __ballot(mine && (!usable || S2 >= (1u << 24)));
    int first = stop ? __ffsll((long long)stop) - 1 : cnt;
    if (first > cnt) first = cnt;
    if (first > from) {
        const uint32_t done = __builtin_amdgcn_readlane(S2, first - 1);
        s = ((uint32_t)es << 23) | (done & 0x7fffffu);
    }
    return first;
}

__global__ __launch_bounds__(SC_WG) void sample_candidates_kernel(const half_t *logits, const float *table, int vocab,
                                                                 int k, uint32_t *out) {
    __shared__ float wave_f[SC_WAVES];
    __shared__ uint32_t wave_u[SC_WAVES];
    __shared__ uint32_t hist[256];
    __shared__ uint32_t wg_counts[2 * SC_MAX_WG];

    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wg = blockIdx.x, nwg = gridDim.x;
    const int seg = wg * SC_WAVES + w, nseg = nwg * SC_WAVES; // this wavefront's range of 512 entries
    const int lo = (wg * SC_WG + t) * 8;                     // this thread's entries [lo, lo + 8)
    uint32_t *ctrl = reinterpret_cast<uint32_t *>(reinterpret_cast<char *>(out) + sc_head_bytes(k));
    // per thread, for the wavefront that walks the ranges: its runs for the guessed exponent and for the next one
    // (4 words), then its 8 table values
    unsigned long long *lane_data = reinterpret_cast<unsigned long long *>(ctrl + C_WORDS);
    const uint16_t *lg = reinterpret_cast<const uint16_t *>(logits);

    // ---- the entries: table value (0 beyond the vocabulary) and order key, in registers from here on ----
    uint32_t key[8];
    float x[8];
    {
        uint16_t b[8];
        if (lo + 8 <= vocab) {
            const uint4_t raw = *reinterpret_cast<const uint4_t *>(lg + lo);
#pragma unroll
            for (int u = 0; u < 8; ++u) b[u] = (uint16_t)(raw[u >> 1] >> ((u & 1) * 16));
        } else {
#pragma unroll
            for (int u = 0; u < 8; ++u) b[u] = lo + u < vocab ? lg[lo + u] : (uint16_t)0xffffu;
        }
        bool bad = false;
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = lo + u < vocab ? table[b[u]] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            bad |= !(x[u] < INFINITY) || x[u] < 0.0f; // NaN logits land here too: the table holds NaN for them
            key[u] = lo + u < vocab ? f16_order_key(b[u]) : 0u;
        }
        if (bad) atomicOr(&ctrl[C_BAD], 1u);
    }
    const int n_own = max(0, min(8, vocab - lo));
    hist[t] = 0;
    __syncthreads();
    {
        uint32_t bin[8];
        bool take[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            bin[u] = key[u] >> 8;
            take[u] = u < n_own;
        }
        hist_add8(hist, bin, take);
    }
    // approximate sum of the wavefront's range: only the exponent guesses use these
    const float own = ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
    const float seg_own = wave_sum(own);
    if (lane == 0) st_agent(&ctrl[C_SEG_SUM + seg], __builtin_bit_cast(uint32_t, seg_own));
    __syncthreads();
    if (hist[t]) atomicAdd(&ctrl[C_HIST1 + t], hist[t]);
    grid_barrier(ctrl, 0, nwg);

    if (ld_agent(&ctrl[C_BAD])) { // the same for every workgroup: nobody waits at a later barrier
        if (wg == 0 && t == 0) {
            out[0] = 0;
            out[1] = 0;
            out[2] = 1; // the host decides on the full vocabulary
            out[3] = 0;
        }
        return;
    }

    // ---- runs: per thread for the guessed exponent and for the next one, per wavefront composed in lane order ----
    {
        float before = 0.0f;
        for (int j = lane; j < seg; j += 64) before += __builtin_bit_cast(float, ld_agent(&ctrl[C_SEG_SUM + j]));
        before = wave_sum(before);
        const int es = seq_guess_exponent(before, seg_own); // 0: the range is expected to change binade
        const int eb = seq_base_exponent(before);
        SeqMap m = {0u, 0u}, m_next = {0u, 0u};
        if (eb) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                seqmap_push(m, __builtin_bit_cast(uint32_t, x[u]), eb);
                seqmap_push(m_next, __builtin_bit_cast(uint32_t, x[u]), eb + 1);
            }
        }
        unsigned long long *mine = lane_data + (size_t)(wg * SC_WG + t) * SC_LANE_WORDS64;
        st_agent64(mine, (unsigned long long)m.a0 | ((unsigned long long)m.a1 << 32));
        st_agent64(mine + 1, (unsigned long long)m_next.a0 | ((unsigned long long)m_next.a1 << 32));
#pragma unroll
        for (int u = 0; u < 8; u += 2)
            st_agent64(mine + 2 + u / 2, (unsigned long long)__builtin_bit_cast(uint32_t, x[u]) |
                                             ((unsigned long long)__builtin_bit_cast(uint32_t, x[u + 1]) << 32));
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            SeqMap o;
            o.a0 = __shfl_down(m.a0, d);
            o.a1 = __shfl_down(m.a1, d);
            if ((lane & (2 * d - 1)) == 0) m = seqmap_compose(m, o);
        }
        if (lane == 0) {
            st_agent(&ctrl[C_SEG_A0 + seg], m.a0);
            st_agent(&ctrl[C_SEG_A1 + seg], m.a1);
            st_agent(&ctrl[C_SEG_ES + seg], (uint32_t)(es == eb ? es : 0));
            st_agent(&ctrl[C_SEG_BASE + seg], (uint32_t)eb);
        }
    }
    grid_barrier(ctrl, 1, nwg);

    // ---- one wavefront walks the ranges in order; all of its lanes hold the same s ----
    if (wg == 0 && w == 0) {
        uint32_t s = 0, one_by_one = 0;
        for (int g0 = 0; g0 < nseg; g0 += 64) {
            const bool have = g0 + lane < nseg && (g0 + lane) * 512 < vocab;
            const uint32_t a0 = have ? ld_agent(&ctrl[C_SEG_A0 + g0 + lane]) : 0u;
            const uint32_t a1 = have ? ld_agent(&ctrl[C_SEG_A1 + g0 + lane]) : 0u;
            const int e = have ? (int)ld_agent(&ctrl[C_SEG_ES + g0 + lane]) : 0;
            const int base = have ? (int)ld_agent(&ctrl[C_SEG_BASE + g0 + lane]) : 0;
            const int cnt = min(64, nseg - g0);
            // ranges expected to change binade are fetched ahead, one at a time, while the walk is busy before them
            unsigned long long expected = __ballot(have && e == 0);
            int ahead = expected ? __ffsll((long long)expected) - 1 : -1;
            ScRange pre;
            if (ahead >= 0) sc_fetch_range(pre, lane_data, g0 + ahead, lane);
            int j = 0;
            while (j < cnt) {
                const int es_now = (int)(s >> 23);
                SeqMap whole = {a0, a1};
                j = sc_apply_prefix(s, whole, have && e != 0 && e == es_now, j, cnt, es_now, lane);
                if (j >= cnt) break;
                if ((g0 + j) * 512 >= vocab) { // nothing but padding
                    ++j;
                    continue;
                }
                // Range j did not go in as a whole (it changes binade, or the guess was off): lane by lane, with a
                // lane's run for the guessed exponent or for the next one where s has that exponent, and the 8
                // values of a lane one after the other where neither applies.
                ScRange cur;
                if (j == ahead) {
                    cur = pre;
                    expected &= ~(1ull << j);
                    ahead = expected ? __ffsll((long long)expected) - 1 : -1;
                    if (ahead >= 0) sc_fetch_range(pre, lane_data, g0 + ahead, lane);
                } else {
                    sc_fetch_range(cur, lane_data, g0 + j, lane);
                }
                const int eb = __builtin_amdgcn_readlane(base, j);
                SeqMap at_base = {(uint32_t)cur.w[0], (uint32_t)(cur.w[0] >> 32)};
                SeqMap at_next = {(uint32_t)cur.w[1], (uint32_t)(cur.w[1] >> 32)};
                uint32_t xq[8];
#pragma unroll
                for (int u = 0; u < 8; u += 2) {
                    xq[u] = (uint32_t)cur.w[2 + u / 2];
                    xq[u + 1] = (uint32_t)(cur.w[2 + u / 2] >> 32);
                }
                int q = 0;
                while (q < 64) {
                    const int eq = (int)(s >> 23);
                    if (eb && eq == eb) q = sc_apply_prefix(s, at_base, true, q, 64, eq, lane);
                    else if (eb && eq == eb + 1) q = sc_apply_prefix(s, at_next, true, q, 64, eq, lane);
                    if (q >= 64) break;
                    ++one_by_one;
                    float f = __builtin_bit_cast(float, s);
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        f = f + __builtin_bit_cast(float, __builtin_amdgcn_readlane(xq[u], q));
                        asm volatile("" : "+v"(f)); // one rounding per addition, in this order
                    }
                    s = __builtin_bit_cast(uint32_t, f);
                    ++q;
                }
                ++j;
            }
        }
        if (lane == 0) {
            st_agent(&ctrl[C_DENOM], s);
            st_agent(&ctrl[C_ONE_BY_ONE], one_by_one);
        }
    }
    hist[t] = ld_agent(&ctrl[C_HIST1 + t]);
    grid_barrier(ctrl, 2, nwg);

    const uint32_t denom_bits = ld_agent(&ctrl[C_DENOM]);
    const float denom = __builtin_bit_cast(float, denom_bits);
    if (!(denom < INFINITY) || !(denom > 0.0f)) {
        if (wg == 0 && t == 0) {
            out[0] = denom_bits;
            out[1] = 0;
            out[2] = 1;
            out[3] = 0;
        }
        return;
    }

    // ---- k-th largest logit by its 16-bit order key: upper byte from the first histogram, then the lower ----
    uint32_t above1, above2;
    const int b1 = pick_bin(hist, (uint32_t)k, above1);
    __syncthreads();
    hist[t] = 0;
    __syncthreads();
    {
        uint32_t bin[8];
        bool take[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            bin[u] = key[u] & 255u;
            take[u] = u < n_own && (int)(key[u] >> 8) == b1;
        }
        hist_add8(hist, bin, take);
    }
    __syncthreads();
    if (hist[t]) atomicAdd(&ctrl[C_HIST2 + t], hist[t]);
    grid_barrier(ctrl, 3, nwg);
    hist[t] = ld_agent(&ctrl[C_HIST2 + t]);
    __syncthreads();
    const int b2 = pick_bin(hist, (uint32_t)k - above1, above2);
    const float p_cut = table[key_to_bits(((uint32_t)b1 << 8) | (uint32_t)b2)] / denom;

    // ---- entries above the cut in any order, then the lowest-indexed entries equal to it, k in all ----
    float p[8];
    uint32_t n_gt = 0, n_eq = 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        p[u] = x[u] / denom;
        n_gt += u < n_own && p[u] > p_cut;
        n_eq += u < n_own && p[u] == p_cut;
    }
    uint32_t wg_gt, wg_eq;
    uint32_t at_gt = block_exclusive<uint32_t>(n_gt, wave_u, wg_gt);
    uint32_t at_eq = block_exclusive<uint32_t>(n_eq, wave_u, wg_eq);
    if (t == 0) {
        st_agent(&ctrl[C_WG_GT + wg], wg_gt);
        st_agent(&ctrl[C_WG_EQ + wg], wg_eq);
    }
    grid_barrier(ctrl, 4, nwg);
    if (t < nwg) {
        wg_counts[t] = ld_agent(&ctrl[C_WG_GT + t]);
        wg_counts[SC_MAX_WG + t] = ld_agent(&ctrl[C_WG_EQ + t]);
    }
    __syncthreads();
    uint32_t total_gt = 0, total_eq = 0;
    for (int j = 0; j < nwg; ++j) {
        if (j == wg) {
            at_gt += total_gt;
            at_eq += total_eq;
        }
        total_gt += wg_counts[j];
        total_eq += wg_counts[SC_MAX_WG + j];
    }
    const bool consistent = total_gt < (uint32_t)k && total_gt + total_eq >= (uint32_t)k; // holds for a monotone table
    const uint32_t room_eq = consistent ? (uint32_t)k - total_gt : 0u;
    if (consistent) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (u >= n_own) continue;
            uint32_t slot = 0xffffffffu;
            if (p[u] > p_cut) slot = at_gt++;
            else if (p[u] == p_cut) {
                if (at_eq < room_eq) slot = total_gt + at_eq;
                ++at_eq;
            }
            if (slot != 0xffffffffu) {
                out[4 + 2 * slot] = __builtin_bit_cast(uint32_t, p[u]);
                out[5 + 2 * slot] = (uint32_t)(lo + u);
            }
        }
    }
    if (wg == 0 && t == 0) {
        out[0] = denom_bits;
        out[1] = consistent ? (uint32_t)k : 0u;
        out[2] = (consistent && !ld_agent(&ctrl[C_TIMEOUT])) ? 0u : 1u;
        out[3] = ld_agent(&ctrl[C_ONE_BY_ONE]);
    }
}

// clears the control block (a kernel rather than a memset so that the pair can be captured into a graph)
__global__ void sample_clear_kernel(uint32_t *ctrl) {
    for (int i = threadIdx.x; i < C_WORDS; i += blockDim.x) ctrl[i] = 0;
}

} // namespace

extern "C" size_t llm_sample_candidates_head_bytes(int k) { return 16 + 8 * (size_t)(k > 0 ? k : 0); }

extern "C" size_t llm_sample_candidates_bytes(int vocab, int k) {
    if (vocab < 1 || k < 1) return 0;
    return sc_head_bytes(k) + sizeof(uint32_t) * C_WORDS + 8 * (size_t)SC_LANE_WORDS64 * sc_workgroups(vocab) * SC_WG;
}

extern "C" int llm_sample_candidates_max_vocab(void) { return SC_MAX_WG * SC_PER_WG; }

extern "C" int llm_sample_candidates(const uint16_t *logits, const float *exp_table, int vocab, int k, void *out,
                                     llm_stream_t stream) {
    LLM_REQUIRE(logits && exp_table && out, "llm_sample_candidates: null pointer");
    LLM_REQUIRE(vocab >= 2 && k >= 1 && k < vocab, "llm_sample_candidates: need 1 <= k < vocab, got k %d vocab %d", k, vocab);
    LLM_REQUIRE(vocab <= SC_MAX_WG * SC_PER_WG, "llm_sample_candidates: vocab %d above the limit of %d", vocab,
                SC_MAX_WG * SC_PER_WG);
    LLM_REQUIRE(aligned16(out) && aligned16(logits), "llm_sample_candidates: logits and out must be 16-byte aligned");
    int cus = 0;
    int rc = llm_cu_count_cached(&cus);
    if (rc != LLM_OK) return rc;
    const int nwg = sc_workgroups(vocab);
    // the workgroups wait for one another inside the kernel: all of them must fit on the device at once
    LLM_REQUIRE(nwg <= cus, "llm_sample_candidates: %d workgroups on a device of %d compute units", nwg, cus);
    uint32_t *ctrl = reinterpret_cast<uint32_t *>(static_cast<char *>(out) + sc_head_bytes(k));
    hipLaunchKernelGGL(sample_clear_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(stream), ctrl);
    LLM_LAUNCH_CHECK("sample_clear_kernel");
    hipLaunchKernelGGL(sample_candidates_kernel, dim3(nwg), dim3(SC_WG), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<const half_t *>(logits), exp_table, vocab, k, static_cast<uint32_t *>(out));
    LLM_LAUNCH_CHECK("sample_candidates_kernel");
    return LLM_OK;
}
