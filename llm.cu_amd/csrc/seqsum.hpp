// The float32 running sum  s = ((x0 + x1) + x2) + ...  of non-negative finite values, bit for bit as a loop
// that adds them one after the other computes it (the reference's softmax denominator,
// src/inference/inference.cu:1049-1056), but with the additions of a whole segment done independently of s.
//
// While s stays inside one binade its unit in the last place u is fixed and s = S*u with an integer S in
// [2^23, 2^24).  Adding x = (X + f)*u, X integer, 0 <= f < 1, under round-to-nearest-even gives S + X when
// f < 1/2, S + X + 1 when f > 1/2, and the even one of the two when f = 1/2: the only thing the step needs to
// know about S is whether it is odd.  A run of additions is therefore a pair (a0, a1), the total increment
// of S for an even and for an odd start, and two runs compose as  c_p = a_p + b_{(p + a_p) mod 2}.  A segment's
// pair needs only the exponent of s, which is guessed from an approximate prefix sum; applying it checks the
// guess against the actual s and that S stays below 2^24 (s only grows, so the end value bounds every
// intermediate one).  Where a check fails the caller adds that segment's values one by one instead, so the
// result never depends on the quality of the guess.
//
// Plain functions on bit patterns, compiled for the device and, by the host-side test, for the CPU.
#pragma once
#include <stdint.h>

#ifndef SEQSUM_FN
#define SEQSUM_FN __host__ __device__ __forceinline__
#endif

struct SeqMap {
    uint32_t a0, a1; // increment of S for an even / an odd S at the start; saturates at SEQ_SAT
};

#define SEQ_SAT (1u << 25) // any increment this large leaves the binade: exact value not needed

// Appends the addition of x (bit pattern of a finite float >= 0) to the run m, for biased exponent es of s.
SEQSUM_FN void seqmap_push(SeqMap &m, uint32_t xbits, int es) {
    const int ex_field = (int)(xbits >> 23);
    const int ex = ex_field ? ex_field : 1;
    const uint32_t mant = (xbits & 0x7fffffu) | (ex_field ? 0x800000u : 0u);
    const int shift = es - ex;
    if (shift < 0) { // x >= 2u * 2^23: the sum leaves the binade for certain
        m.a0 = m.a1 = SEQ_SAT;
        return;
    }
    if (shift > 24 || mant == 0) return; // less than half a unit: s unchanged
    const uint32_t X = shift < 24 ? mant >> shift : 0u;
    uint32_t c0 = 0, c1 = 0;
    if (shift > 0) {
        const uint32_t rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half) {
            c0 = c1 = 1;
        } else if (rem == half) { // tie: up exactly when S + X is odd
            c0 = (m.a0 + X) & 1u;
            c1 = (1u + m.a1 + X) & 1u;
        }
    }
    m.a0 += X + c0;
    m.a1 += X + c1;
    if (m.a0 > SEQ_SAT) m.a0 = SEQ_SAT;
    if (m.a1 > SEQ_SAT) m.a1 = SEQ_SAT;
}

// first, then second
SEQSUM_FN SeqMap seqmap_compose(SeqMap first, SeqMap second) {
    SeqMap c;
    c.a0 = first.a0 + ((first.a0 & 1u) ? second.a1 : second.a0);
    c.a1 = first.a1 + (((1u + first.a1) & 1u) ? second.a1 : second.a0);
    if (c.a0 > SEQ_SAT) c.a0 = SEQ_SAT;
    if (c.a1 > SEQ_SAT) c.a1 = SEQ_SAT;
    return c;
}

// Applies a run computed for exponent es to s.  False (s untouched) when s is not a normal number of that
// exponent or the run carries it out of the binade.
SEQSUM_FN bool seqmap_apply(uint32_t &sbits, SeqMap m, int es) {
    if (es < 1 || es > 253 || (int)(sbits >> 23) != es) return false;
    const uint32_t S = (sbits & 0x7fffffu) | 0x800000u;
    const uint32_t S2 = S + ((S & 1u) ? m.a1 : m.a0);
    if (S2 >= (1u << 24)) return false;
    sbits = ((uint32_t)es << 23) | (S2 & 0x7fffffu);
    return true;
}

// Exponent to compute a segment's run for, from an approximate sum before it and an approximate sum of it;
// 0 (never valid) when the approximation says that s is not yet normal or changes binade inside the segment.
SEQSUM_FN int seq_guess_exponent(float before, float own) {
    const float after = before + own * 1.0001f;
    const uint32_t b = __builtin_bit_cast(uint32_t, before), a = __builtin_bit_cast(uint32_t, after);
    const int eb = (int)(b >> 23), ea = (int)(a >> 23);
    return (eb == ea && eb >= 1 && eb <= 253) ? eb : 0;
}

// Exponent of the approximate sum before a segment, for runs that are computed for it and for the next one
// (what a walk through a segment that changes binade falls back on); 0 when that sum is not a normal number.
SEQSUM_FN int seq_base_exponent(float before) {
    const int eb = (int)(__builtin_bit_cast(uint32_t, before) >> 23);
    return (eb >= 1 && eb <= 252) ? eb : 0;
}
