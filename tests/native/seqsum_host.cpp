// CPU build of llm.cu_amd/csrc/seqsum.hpp for tests/test_seqsum.py: the segment scheme of the device
// kernel (approximate prefix -> exponent guess -> per-segment run -> sequential application with
// fall-back), driven over a host array.
#include <cstdint>
#include <cstring>
#include <vector>
#define SEQSUM_FN static inline
#include "seqsum.hpp"

static uint32_t bits_of(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

extern "C" float seqsum_segments(const float *x, int n, int seg_len, int *n_sequential) {
    const int n_seg = (n + seg_len - 1) / seg_len;
    std::vector<float> own(n_seg), before(n_seg);
    for (int j = 0; j < n_seg; ++j) {
        float a = 0.0f;
        for (int i = j * seg_len; i < n && i < (j + 1) * seg_len; ++i) a += x[i];
        own[j] = a;
    }
    // a deliberately different summation order from the exact one: pairs of segments first
    float run = 0.0f;
    for (int j = 0; j < n_seg; j += 2) {
        before[j] = run;
        if (j + 1 < n_seg) before[j + 1] = run + own[j];
        run += own[j] + (j + 1 < n_seg ? own[j + 1] : 0.0f);
    }
    std::vector<SeqMap> maps(n_seg);
    std::vector<int> es(n_seg);
    for (int j = 0; j < n_seg; ++j) {
        es[j] = seq_guess_exponent(before[j], own[j]);
        SeqMap m = {0, 0};
        if (es[j])
            for (int i = j * seg_len; i < n && i < (j + 1) * seg_len; ++i) seqmap_push(m, bits_of(x[i]), es[j]);
        maps[j] = m;
    }
    uint32_t s = 0;
    int fallbacks = 0;
    for (int j = 0; j < n_seg; ++j) {
        if (seqmap_apply(s, maps[j], es[j])) continue;
        ++fallbacks;
        float f;
        memcpy(&f, &s, 4);
        for (int i = j * seg_len; i < n && i < (j + 1) * seg_len; ++i) f = f + x[i];
        s = bits_of(f);
    }
    if (n_sequential) *n_sequential = fallbacks;
    float f;
    memcpy(&f, &s, 4);
    return f;
}

// pairs composed before they are applied (the order a tree of lanes would use)
extern "C" float seqsum_composed(const float *x, int n, int es, int *ok) {
    std::vector<SeqMap> m(n);
    for (int i = 0; i < n; ++i) {
        m[i] = SeqMap{0, 0};
        seqmap_push(m[i], bits_of(x[i + 1]), es);
    }
    for (int stride = 1; stride < n; stride *= 2)
        for (int i = 0; i + stride < n; i += 2 * stride) m[i] = seqmap_compose(m[i], m[i + stride]);
    uint32_t s = bits_of(x[0]);
    *ok = seqmap_apply(s, m[0], es) ? 1 : 0;
    float f;
    memcpy(&f, &s, 4);
    return f;
}
