// Host sampler of the reference (src/inference/inference.cu:1030-1161), kept call for call:
// temperature softmax over the fp16 logits without max subtraction, a descending qsort of the whole
// vocabulary, a top-k pass whose renormalisation of the first k entries stays in the array and whose
// draw is thrown away, then the top-p pass that picks the token.  Randomness is the C library's rand(),
// unseeded in the reference, so the stream is shared with every other caller in the process.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>

#include "../common/fail.h"
#include "llama3_host.h"
#include "sampler.h"

// Settings of the reference-named entry points below, which take no settings argument (the reference
// fixes them at compile time).  A CudaCache carries its own SamplerParams: inference() never reads these.
static SamplerParams g_params; // VOCAB_SIZE, TEMPERATURE, TOP_K, TOP_P of inference.cu:24-29

// __half2float: exact widening of an fp16 bit pattern
static float half_to_float(llm_half h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
    if (exp == 0x1Fu) {
        bits = sign | 0x7F800000u | (man << 13);
    } else if (exp != 0) {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    } else if (man == 0) {
        bits = sign;
    } else { // subnormal: normalise
        int e = -1;
        do {
            man <<= 1;
            ++e;
        } while (!(man & 0x400u));
        bits = sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3FFu) << 13);
    }
    float f;
    memcpy(&f, &bits, sizeof f);
    return f;
}

extern "C" int _compare_desc(const void *a, const void *b);

// inference.cu:1043-1072
static ProbIndex *softmax_sorted(int vocab, float *tensor, const llm_half *half_tensor, float temperature) {
    ProbIndex *arr = (ProbIndex *)malloc((size_t)vocab * sizeof(ProbIndex));
    if (!arr) llama3_fail("temperature_softmax: out of memory");
    float cumsum = 0.0f;
    for (int i = 0; i < vocab; ++i) {
        const float scaled = half_to_float(half_tensor[i]) / temperature;
        tensor[i] = expf(scaled); // the reference's exp(float) in a C++ translation unit is the float overload (inference.cu:1048)
        cumsum += tensor[i];
    }
    for (int i = 0; i < vocab; ++i) {
        tensor[i] /= cumsum;
        arr[i].probability = tensor[i];
        arr[i].index = i;
    }
    qsort(arr, (size_t)vocab, sizeof(ProbIndex), _compare_desc);
    return arr;
}

// inference.cu:1086-1113
static int top_k_pick(int vocab, ProbIndex *arr, int k) {
    if (k <= 0) return arr[rand() % vocab].index;
    if (k > vocab) k = vocab;
    float sum = 0.0f;
    for (int i = 0; i < k; ++i) sum += arr[i].probability;
    for (int i = 0; i < k; ++i) arr[i].probability /= sum;
    const float r = (float)rand() / (float)RAND_MAX;
    float cumulative = 0.0f;
    for (int i = 0; i < k; ++i) {
        cumulative += arr[i].probability;
        if (r < cumulative) return arr[i].index;
    }
    return arr[0].index;
}

// inference.cu:1115-1161.  n: entries of arr that exist (the whole vocabulary in the reference's flow).
static int top_p_pick(int vocab, ProbIndex *arr, int n, float p) {
    if (p <= 0.0f) return arr[rand() % vocab].index;
    if (p > 1.0f) p = 1.0f;
    float cumulative = 0.0f;
    int cutoff = 0;
    for (; cutoff < n; ++cutoff) {
        cumulative += arr[cutoff].probability;
        if (cumulative >= p) break;
    }
    const float sum = cumulative;
    if (cutoff >= n) cutoff = n - 1;
    for (int i = 0; i <= cutoff; ++i) arr[i].probability /= sum;
    const float r = (float)rand() / (float)RAND_MAX;
    cumulative = 0.0f;
    for (int i = 0; i <= cutoff; ++i) {
        cumulative += arr[i].probability;
        if (r < cumulative) return arr[i].index;
    }
    return arr[0].index;
}

int sampler_draw_reference(const SamplerParams &sp, float *tensor, const llm_half *half_tensor) {
    ProbIndex *arr = softmax_sorted(sp.vocab, tensor, half_tensor, sp.temperature);
    int selected = top_k_pick(sp.vocab, arr, sp.top_k);
    selected = top_p_pick(sp.vocab, arr, sp.vocab, sp.top_p);
    free(arr);
    return selected;
}

bool sampler_head_suffices(const SamplerParams &sp) {
    return sp.top_k > 0 && sp.top_k < sp.vocab && sp.top_p > 0.0f && sp.top_p <= 0.99f;
}

static bool prob_before(const ProbIndex &a, const ProbIndex &b) {
    return a.probability > b.probability || (a.probability == b.probability && a.index < b.index);
}

bool sampler_fill_exp_table(float temperature, float *table) {
    for (uint32_t b = 0; b < 65536u; ++b) table[b] = expf(half_to_float((llm_half)b) / temperature);
    // walk the finite patterns in value order: negative ones from the largest magnitude down, then the positive
    float prev = -INFINITY;
    bool monotone = true;
    for (int i = 0; i < 2 * 0x7c00 && monotone; ++i) {
        const uint32_t b = i < 0x7c00 ? 0x8000u + (uint32_t)(0x7bff - i) : (uint32_t)(i - 0x7c00);
        const float v = table[b];
        if (v != v || v < prev) monotone = false;
        prev = v;
    }
    return monotone;
}

int sampler_draw_from_head(const SamplerParams &sp, ProbIndex *head, int k) {
    std::sort(head, head + k, prob_before);
    (void)top_k_pick(sp.vocab, head, k); // renormalises the head and consumes one rand(), result unused
    return top_p_pick(sp.vocab, head, k, sp.top_p);
}

// Same result without sorting the vocabulary.  After the top-k pass has renormalised the first k
// entries they sum to 1 up to rounding, so for top_p below that sum the top-p pass never looks past
// entry k-1: only the k largest probabilities, in the order qsort leaves them, matter.  glibc's qsort
// is a merge sort (stable) whenever it can allocate its buffer, so equal probabilities stay in index
// order; partial_sort with the index as second key reproduces that head exactly.  Falls back to the
// full path for settings where the tail of the array is reachable.
int sampler_draw(const SamplerParams &sp, float *tensor, const llm_half *half_tensor) {
    const int k = sp.top_k, vocab = sp.vocab;
    if (!sampler_head_suffices(sp)) return sampler_draw_reference(sp, tensor, half_tensor);
    // the exponentials are independent (any thread gives the same bits); their sum is taken afterwards in
    // index order, as the reference's single loop does
    const float temperature = sp.temperature;
#pragma omp parallel for schedule(static)
    for (int i = 0; i < vocab; ++i) tensor[i] = expf(half_to_float(half_tensor[i]) / temperature);
    float cumsum = 0.0f;
    for (int i = 0; i < vocab; ++i) cumsum += tensor[i];
#pragma omp parallel for schedule(static)
    for (int i = 0; i < vocab; ++i) tensor[i] /= cumsum;
    // NaN probabilities (exp overflow) defeat every comparison: let the reference path decide
    if (!(cumsum < INFINITY) || !(cumsum > 0.0f)) return sampler_draw_reference(sp, tensor, half_tensor);
    // k largest by (probability desc, index asc): threshold pass, then a sort of the few survivors
    const int cap = 2 * k + 64;
    ProbIndex *head = (ProbIndex *)malloc((size_t)cap * sizeof(ProbIndex));
    if (!head) llama3_fail("sample_next_token: out of memory");
    int n = 0;
    float floor_p = -1.0f; // entries below the current k-th best cannot enter the head
    auto better = [](const ProbIndex &a, const ProbIndex &b) {
        return a.probability > b.probability || (a.probability == b.probability && a.index < b.index);
    };
    for (int i = 0; i < vocab; ++i) {
        const float p = tensor[i];
        if (p < floor_p) continue; // ties with the floor come later in index order only if p == floor: keep them
        head[n].probability = p;
        head[n].index = i;
        if (++n == cap) {
            std::partial_sort(head, head + k, head + n, better);
            n = k;
            floor_p = head[k - 1].probability;
        }
    }
    if (n > k) {
        std::partial_sort(head, head + k, head + n, better);
        n = k;
    } else {
        std::sort(head, head + n, better);
    }
    int selected = top_k_pick(vocab, head, k);
    selected = top_p_pick(vocab, head, k, sp.top_p);
    free(head);
    return selected;
}

extern "C" {

void llama3_sampler_config(int vocab, float temperature, int top_k, float top_p) {
    if (vocab < 1) llama3_fail("llama3_sampler_config: vocab must be positive");
    g_params.vocab = vocab;
    g_params.temperature = temperature;
    g_params.top_k = top_k;
    g_params.top_p = top_p;
}

// inference.cu:1074-1084
int _compare_desc(const void *a, const void *b) {
    const ProbIndex *pa = (const ProbIndex *)a, *pb = (const ProbIndex *)b;
    if (pa->probability < pb->probability) return 1;
    if (pa->probability > pb->probability) return -1;
    return 0;
}

// The sampler with its settings as arguments (no process-wide state is read or written).
int llama3_sample_with(int vocab, float temperature, int top_k, float top_p, float *tensor, llm_half *half_tensor) {
    if (vocab < 1) llama3_fail("llama3_sample_with: vocab must be positive");
    SamplerParams sp;
    sp.vocab = vocab;
    sp.temperature = temperature;
    sp.top_k = top_k;
    sp.top_p = top_p;
    return sampler_draw(sp, tensor, half_tensor);
}

// inference.cu:1043-1072
ProbIndex *temperature_softmax(float *tensor, llm_half *half_tensor, float temperature) {
    return softmax_sorted(g_params.vocab, tensor, half_tensor, temperature);
}

// inference.cu:1086-1113
int top_k_sampling(ProbIndex *arr, int k) { return top_k_pick(g_params.vocab, arr, k); }

// inference.cu:1115-1161
int top_p_sampling(ProbIndex *arr, float p) { return top_p_pick(g_params.vocab, arr, g_params.vocab, p); }

// inference.cu:1030-1041, call for call (a full qsort of the vocabulary per token: ~10 ms at 128256)
int sample_next_token_reference(float *tensor, llm_half *half_tensor) {
    return sampler_draw_reference(g_params, tensor, half_tensor);
}

int sample_next_token(float *tensor, llm_half *half_tensor) { return sampler_draw(g_params, tensor, half_tensor); }

} // extern "C"
