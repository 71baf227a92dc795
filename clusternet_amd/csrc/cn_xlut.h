// Per-call encoder table of compression_8bit, shared by the device build kernel and a host build
// used by the CPU tests (plain inline C++, compiled by hipcc for both sides and by nothing else).
//
// For a fixed precision the code of x is a step function of |x| (IEEE division and the reference's
// search are both monotone in |x|) with the sign of x / precision on top.  The table is indexed by
// the leading 17 bits of |x| (exponent and 8 mantissa bits): every bucket stores the code below and
// above the one step it can contain, for either sign of x, and the first bit pattern that takes
// the upper code.  All entries come from the literal procedure (encode_exact), evaluated at the
// bucket ends and, where they differ, at the points of a binary search, so the table reproduces
// the literal procedure for every input by construction: no approximate quotient, no guard band,
// no restriction on the precision.  Buckets of the logarithmic range are 0.4 % wide and the
// codebook's steps are at least 0.8 % apart, so a bucket holds at most one step; where that fails
// (denormal inputs under a tiny precision) or the fixed-size table does not cover the code range,
// the build reports it and the encoder evaluates the literal procedure for every element.
#pragma once

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define CN_HD __host__ __device__ inline
#else
#define CN_HD inline
#endif

namespace cn {

constexpr int kXShift = 15;        // |x| pattern >> 15 = bucket number (0 .. 0xffff)
constexpr int kXBuckets = 5056;    // 19.75 binades; the coded range 1.5e-6 .. 0.9957 spans 19.34
constexpr int kXEntries = kXBuckets + 2;  // a sentinel below and above

struct XEntry {
    uint32_t boundary;  // first |x| pattern that takes the `above` codes
    uint32_t codes;     // bytes: below (x >= 0), above (x >= 0), below (x < 0), above (x < 0)
};

CN_HD float x_from_bits(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }
CN_HD uint32_t x_to_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }

// The reference procedure, element by element (kCompression_8bit, source/clusterKernels.cu:1163-1232):
// IEEE division, sign split, two threshold exits, 6-step pivot search over the table, two-candidate
// pick.  `slot` is a 128-entry copy of the table whose entry 126 holds 1.0f.
CN_HD uint32_t encode_exact(float x, float precision, const float *slot) {
    float a = x / precision;
    uint32_t neg = 0;
    if (a < 0.0f) { neg = 0x80u; a = -a; }
    if (a < 0.0000015f) return 254u;
    if (a > 0.995703f) return 127u | neg;
    int lo = 0, hi = 125, p = 63;
    for (int step = 32; step > 0; step >>= 1) {
        if (a > slot[p]) { lo = p; p += step; }
        else             { hi = p; p -= step; }
    }
    const float dp = slot[p] - a;
    int c;
    if (lo == p) c = ((dp < 0 ? -dp : dp) < (slot[hi] - a)) ? p : hi;
    else { const float dl = slot[lo] - a; c = (dp < (dl < 0 ? -dl : dl)) ? p : lo; }
    return (uint32_t)c | neg;
}

// Bucket number of table entry 1 for this precision: one bucket below the bucket of 1.4e-6 |p|
// (the lower code threshold is 1.5e-6 |p|), 0 when that underflows.  Meaningless for a precision
// that is zero, infinite or NaN; the checks in xlut_entry then report the table as unusable.
CN_HD uint32_t xlut_first(float precision) {
    const float t = (precision < 0 ? -precision : precision) * 1.4e-6f;
    const uint32_t b = (x_to_bits(t) & 0x7fffffffu) >> kXShift;
    return b > 0 ? b - 1 : 0;
}

CN_HD uint32_t pack_codes(uint32_t below_pos, uint32_t above_pos, uint32_t below_neg, uint32_t above_neg) {
    return below_pos | (above_pos << 8) | (below_neg << 16) | (above_neg << 24);
}

// Entry `index` (0 .. kXEntries - 1) of the table for `precision`.  *unusable is set when the entry
// cannot represent its range exactly.
CN_HD XEntry xlut_entry(int index, float precision, const float *slot, bool *unusable) {
    const uint32_t first = xlut_first(precision);
    const uint32_t kSign = 0x80000000u;
    *unusable = false;
    if (index == 0) {
        // everything below bucket `first`: must be code 254 throughout, i.e. at its largest pattern
        if (first > 0) {
            const uint32_t top = (first << kXShift) - 1;
            if (encode_exact(x_from_bits(top), precision, slot) != 254u ||
                encode_exact(x_from_bits(top | kSign), precision, slot) != 254u) *unusable = true;
        }
        return XEntry{0xffffffffu, pack_codes(254, 254, 254, 254)};
    }
    if (index == kXEntries - 1) {
        // everything above the last bucket: one code up to infinity, then the code of a NaN
        const uint64_t start = ((uint64_t)first + kXBuckets) << kXShift;
        const uint32_t c_nan = encode_exact(x_from_bits(0x7fc00000u), precision, slot);
        const uint32_t n_nan = encode_exact(x_from_bits(0xffc00000u), precision, slot);
        if (start > 0x7f800000u) return XEntry{0u, pack_codes(c_nan, c_nan, n_nan, n_nan)};  // only NaNs left
        const uint32_t c0 = encode_exact(x_from_bits((uint32_t)start), precision, slot);
        const uint32_t n0 = encode_exact(x_from_bits((uint32_t)start | kSign), precision, slot);
        if (c0 != encode_exact(x_from_bits(0x7f800000u), precision, slot) ||
            n0 != encode_exact(x_from_bits(0xff800000u), precision, slot)) *unusable = true;
        return XEntry{0x7f800001u, pack_codes(c0, c_nan, n0, n_nan)};
    }
    const uint64_t bucket = (uint64_t)first + (uint32_t)(index - 1);
    if (bucket > 0xffffu) return XEntry{0xffffffffu, 0u};  // beyond the last bit pattern: never indexed
    const uint32_t lo = (uint32_t)bucket << kXShift, hi = lo + ((1u << kXShift) - 1);
    const uint32_t c_lo = encode_exact(x_from_bits(lo), precision, slot);
    const uint32_t c_hi = encode_exact(x_from_bits(hi), precision, slot);
    const uint32_t n_lo = encode_exact(x_from_bits(lo | kSign), precision, slot);
    const uint32_t n_hi = encode_exact(x_from_bits(hi | kSign), precision, slot);
    if (c_lo == c_hi && n_lo == n_hi) return XEntry{lo, pack_codes(c_lo, c_lo, n_lo, n_lo)};
    // smallest pattern in (lo, hi] whose code differs from the code at lo
    uint32_t below = lo, above = hi;  // code(below) == c_lo, code(above) != c_lo
    if (c_lo == c_hi) { *unusable = true; return XEntry{lo, pack_codes(c_lo, c_lo, n_lo, n_lo)}; }
    while (above - below > 1) {
        const uint32_t mid = below + (above - below) / 2;
        if (encode_exact(x_from_bits(mid), precision, slot) == c_lo) below = mid; else above = mid;
    }
    // one step only: the code right above the step is already the code at the bucket's end, and
    // the negative side steps at the same pattern
    if (encode_exact(x_from_bits(above), precision, slot) != c_hi ||
        encode_exact(x_from_bits(below | kSign), precision, slot) != n_lo ||
        encode_exact(x_from_bits(above | kSign), precision, slot) != n_hi) *unusable = true;
    return XEntry{above, pack_codes(c_lo, c_hi, n_lo, n_hi)};
}

// Table index of a bit pattern.
CN_HD int xlut_index(uint32_t magnitude_bits, uint32_t first) {
    int i = (int)(magnitude_bits >> kXShift) - (int)first + 1;
    i = i < 0 ? 0 : i;
    return i > kXEntries - 1 ? kXEntries - 1 : i;
}

// Code of the pattern `bits` from its table entry.
CN_HD uint32_t xlut_code(uint32_t bits, XEntry e) {
    const uint32_t mag = bits & 0x7fffffffu;
    const uint32_t sel = ((bits >> 31) << 4) | ((mag >= e.boundary ? 1u : 0u) << 3);
    return (e.codes >> sel) & 0xffu;
}

}  // namespace cn
