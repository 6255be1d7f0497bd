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

static int g_vocab = 128256;           // VOCAB_SIZE, inference.cu:24
static float g_temperature = 0.7f;     // TEMPERATURE, inference.cu:27
static int g_top_k = 50;               // TOP_K, inference.cu:28
static float g_top_p = 0.9f;           // TOP_P, inference.cu:29

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

extern "C" {

void llama3_sampler_config(int vocab, float temperature, int top_k, float top_p) {
    if (vocab < 1) llama3_fail("llama3_sampler_config: vocab must be positive");
    g_vocab = vocab;
    g_temperature = temperature;
    g_top_k = top_k;
    g_top_p = top_p;
}

// inference.cu:1074-1084
int _compare_desc(const void *a, const void *b) {
    const ProbIndex *pa = (const ProbIndex *)a, *pb = (const ProbIndex *)b;
    if (pa->probability < pb->probability) return 1;
    if (pa->probability > pb->probability) return -1;
    return 0;
}

// inference.cu:1043-1072
ProbIndex *temperature_softmax(float *tensor, llm_half *half_tensor, float temperature) {
    ProbIndex *arr = (ProbIndex *)malloc((size_t)g_vocab * sizeof(ProbIndex));
    if (!arr) llama3_fail("temperature_softmax: out of memory");
    float cumsum = 0.0f;
    for (int i = 0; i < g_vocab; ++i) {
        const float scaled = half_to_float(half_tensor[i]) / temperature;
        tensor[i] = expf(scaled);
        cumsum += tensor[i];
    }
    for (int i = 0; i < g_vocab; ++i) {
        tensor[i] /= cumsum;
        arr[i].probability = tensor[i];
        arr[i].index = i;
    }
    qsort(arr, (size_t)g_vocab, sizeof(ProbIndex), _compare_desc);
    return arr;
}

// inference.cu:1086-1113
int top_k_sampling(ProbIndex *arr, int k) {
    if (k <= 0) return arr[rand() % g_vocab].index;
    if (k > g_vocab) k = g_vocab;
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

// inference.cu:1115-1161
int top_p_sampling(ProbIndex *arr, float p) {
    if (p <= 0.0f) return arr[rand() % g_vocab].index;
    if (p > 1.0f) p = 1.0f;
    float cumulative = 0.0f;
    int cutoff = 0;
    for (; cutoff < g_vocab; ++cutoff) {
        cumulative += arr[cutoff].probability;
        if (cumulative >= p) break;
    }
    const float sum = cumulative;
    if (cutoff >= g_vocab) cutoff = g_vocab - 1;
    for (int i = 0; i <= cutoff; ++i) arr[i].probability /= sum;
    const float r = (float)rand() / (float)RAND_MAX;
    cumulative = 0.0f;
    for (int i = 0; i <= cutoff; ++i) {
        cumulative += arr[i].probability;
        if (r < cumulative) return arr[i].index;
    }
    return arr[0].index;
}

// inference.cu:1030-1041, call for call (a full qsort of the vocabulary per token: ~10 ms at 128256)
int sample_next_token_reference(float *tensor, llm_half *half_tensor) {
    ProbIndex *arr = temperature_softmax(tensor, half_tensor, g_temperature);
    int selected = top_k_sampling(arr, g_top_k);
    selected = top_p_sampling(arr, g_top_p);
    free(arr);
    return selected;
}

// Same result without sorting the vocabulary.  After top_k_sampling() has renormalised the first k
// entries they sum to 1 up to rounding, so for top_p below that sum top_p_sampling() never looks past
// entry k-1: only the k largest probabilities, in the order qsort leaves them, matter.  glibc's qsort
// is a merge sort (stable) whenever it can allocate its buffer, so equal probabilities stay in index
// order; partial_sort with the index as second key reproduces that head exactly.  Falls back to the
// full path for settings where the tail of the array is reachable.
int sample_next_token(float *tensor, llm_half *half_tensor) {
    const int k = g_top_k;
    if (k <= 0 || k >= g_vocab || !(g_top_p > 0.0f) || g_top_p > 0.99f)
        return sample_next_token_reference(tensor, half_tensor);
    // the exponentials are independent (any thread gives the same bits); their sum is taken afterwards in
    // index order, as the reference's single loop does
    const int vocab = g_vocab;
    const float temperature = g_temperature;
#pragma omp parallel for schedule(static)
    for (int i = 0; i < vocab; ++i) tensor[i] = expf(half_to_float(half_tensor[i]) / temperature);
    float cumsum = 0.0f;
    for (int i = 0; i < vocab; ++i) cumsum += tensor[i];
#pragma omp parallel for schedule(static)
    for (int i = 0; i < vocab; ++i) tensor[i] /= cumsum;
    // NaN probabilities (exp overflow) defeat every comparison: let the reference path decide
    if (!(cumsum < INFINITY) || !(cumsum > 0.0f)) return sample_next_token_reference(tensor, half_tensor);
    // k largest by (probability desc, index asc): threshold pass, then a sort of the few survivors
    ProbIndex *head = (ProbIndex *)malloc((size_t)(2 * k + 64) * sizeof(ProbIndex));
    if (!head) llama3_fail("sample_next_token: out of memory");
    int n = 0;
    const int cap = 2 * k + 64;
    float floor_p = -1.0f; // entries below the current k-th best cannot enter the head
    auto better = [](const ProbIndex &a, const ProbIndex &b) {
        return a.probability > b.probability || (a.probability == b.probability && a.index < b.index);
    };
    for (int i = 0; i < g_vocab; ++i) {
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
    int selected = top_k_sampling(head, k);
    selected = top_p_sampling(head, g_top_p);
    free(head);
    return selected;
}

} // extern "C"
