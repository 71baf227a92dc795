// Encoder table of compression_8bit: construction and lookup, shared by the device kernel (every
// workgroup builds the table for the call's precision in LDS) and by a host build used by the CPU
// tests.  Plain inline C++.
//
// For a fixed precision the code of x is a step function of |x| (IEEE division and the reference's
// search are both monotone in |x|) with the sign of x / precision on top.  The table is indexed by
// the leading 17 bits of |x| (exponent and 8 mantissa bits): every bucket stores the code below and
// above the one step it can contain, for either sign of x, and the first bit pattern that takes
// the upper code.  The steps come from evaluations of the literal procedure (encode_exact) at precision 1,
// where the quotient is |x| itself, and are carried to another precision by the one operation through
// which the procedure sees x, the IEEE division (xlut_locate_step); the two sentinel entries are literal
// evaluations at the precision itself.  No approximate quotient, no guard band, no restriction on the
// precision.  Buckets of the logarithmic range are 0.4 % wide
// and the codebook's steps are at least 0.8 % apart, so a bucket holds at most one step; where that
// fails (denormal inputs under a tiny precision), where a step cannot be pinned down or where the
// fixed-size table does not cover the coded range, the build says so and the encoder evaluates the
// literal procedure for every element instead.
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
    // Written without branches (selects only) so that independent evaluations overlap on the device;
    // the two threshold exits of the reference are applied last, which gives the same result because
    // the search itself has no side effects.
    float a = x / precision;
    const uint32_t neg = (a < 0.0f) ? 0x80u : 0u;
    a = (a < 0.0f) ? -a : a;
    int lo = 0, hi = 125, p = 63;
#if defined(__HIPCC__)
#pragma unroll
#endif
    for (int step = 32; step > 0; step >>= 1) {
        const bool up = a > slot[p];
        lo = up ? p : lo;
        hi = up ? hi : p;
        p = up ? p + step : p - step;
    }
    const float dp = slot[p] - a, dh = slot[hi] - a, dl = slot[lo] - a;
    const float adp = dp < 0 ? -dp : dp, adl = dl < 0 ? -dl : dl;
    const int c_first = (adp < dh) ? p : hi;   // lo == p
    const int c_other = (dp < adl) ? p : lo;
    uint32_t code = (uint32_t)((lo == p) ? c_first : c_other) | neg;
    code = (a > 0.995703f) ? (127u | neg) : code;
    code = (a < 0.0000015f) ? 254u : code;
    return code;
}

// N evaluations of encode_exact, written level by level so that the N table reads of a search level
// are independent of each other (a single evaluation is a chain of seven dependent reads).
template <int N>
CN_HD void encode_exact_many(const uint32_t (&bits)[N], float precision, const float *slot, uint32_t (&code)[N]) {
    float a[N];
    uint32_t neg[N];
    int lo[N], hi[N], p[N];
    for (int j = 0; j < N; ++j) {
        const float q = x_from_bits(bits[j]) / precision;
        neg[j] = (q < 0.0f) ? 0x80u : 0u;
        a[j] = (q < 0.0f) ? -q : q;
        lo[j] = 0; hi[j] = 125; p[j] = 63;
    }
    for (int step = 32; step > 0; step >>= 1) {
        float t[N];
        for (int j = 0; j < N; ++j) t[j] = slot[p[j]];
        for (int j = 0; j < N; ++j) {
            const bool up = a[j] > t[j];
            lo[j] = up ? p[j] : lo[j];
            hi[j] = up ? hi[j] : p[j];
            p[j] = up ? p[j] + step : p[j] - step;
        }
    }
    float tp[N], th[N], tl[N];
    for (int j = 0; j < N; ++j) { tp[j] = slot[p[j]]; th[j] = slot[hi[j]]; tl[j] = slot[lo[j]]; }
    for (int j = 0; j < N; ++j) {
        const float dp = tp[j] - a[j], dh = th[j] - a[j], dl = tl[j] - a[j];
        const float adp = dp < 0 ? -dp : dp, adl = dl < 0 ? -dl : dl;
        const int c_first = (adp < dh) ? p[j] : hi[j];
        const int c_other = (dp < adl) ? p[j] : lo[j];
        uint32_t c = (uint32_t)((lo[j] == p[j]) ? c_first : c_other) | neg[j];
        c = (a[j] > 0.995703f) ? (127u | neg[j]) : c;
        c = (a[j] < 0.0000015f) ? 254u : c;
        code[j] = c;
    }
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
            const uint32_t in[2] = {top, top | kSign};
            uint32_t c[2];
            encode_exact_many<2>(in, precision, slot, c);
            if (c[0] != 254u || c[1] != 254u) *unusable = true;
        }
        return XEntry{0xffffffffu, pack_codes(254, 254, 254, 254)};
    }
    if (index == kXEntries - 1) {
        // everything above the last bucket: one code up to infinity, then the code of a NaN
        const uint64_t start64 = ((uint64_t)first + kXBuckets) << kXShift;
        const uint32_t start = start64 > 0x7f800000u ? 0x7f800000u : (uint32_t)start64;
        const uint32_t in[6] = {0x7fc00000u, 0xffc00000u, start, start | kSign, 0x7f800000u, 0xff800000u};
        uint32_t c[6];
        encode_exact_many<6>(in, precision, slot, c);
        if (start64 > 0x7f800000u) return XEntry{0u, pack_codes(c[0], c[0], c[1], c[1])};  // only NaNs left
        if (c[2] != c[4] || c[3] != c[5]) *unusable = true;
        return XEntry{0x7f800001u, pack_codes(c[2], c[0], c[3], c[1])};
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

// ---- building the table from the list of steps --------------------------------------------------
// At precision 1 the table above is built bucket by bucket (on the host, once).  Its steps - the
// smallest quotient pattern S that takes the upper code, with the two magnitude codes - are the same
// for every precision, because the code depends on x only through fl(|x| / |p|).  For another
// precision the step sits at the smallest |x| with fl(|x| / |p|) >= S, within two patterns of
// fl(S |p|): a workgroup finds all steps with ten divisions each and fills the buckets between them,
// which is cheap enough to do in every workgroup instead of sharing a table.
struct XStep {
    uint32_t boundary;  // S: smallest quotient pattern that takes `above`
    uint32_t codes;     // below | above << 8, magnitude codes (0 .. 127 or 254)
};
constexpr int kXMaxSteps = 160;

CN_HD uint32_t magnitude_code(uint32_t c) { return c == 254u ? 254u : (c & 0x7fu); }

// Step `s` under `precision`: its entry (boundary in |x| patterns, the four codes).  The literal procedure
// looks at x only through the quotient x / precision: it takes the sign from it, and the magnitude code is a
// step function of a = |x / precision| whose steps (found once, at precision 1, where a = |x| exactly) are
// the S of the list.  IEEE division is monotone in |x| and symmetric in the signs, so under another precision
// the step sits at the smallest |x| pattern with fl(|x| / |p|) >= S, within two patterns of fl(S |p|): ten
// divisions around that estimate find it, and the four codes follow from the step's two magnitude codes and
// the sign of the precision (254 carries no sign: the reference returns it before the sign is applied).
// False when the step cannot be pinned down (estimate out of range, no change of sides among the ten).
CN_HD bool xlut_locate_step(XStep s, float precision, const float * /*slot*/, XEntry *entry) {
    const float ap = precision < 0 ? -precision : precision;
    const uint32_t est = x_to_bits(x_from_bits(s.boundary) * ap);
    if (!(est >= 16u && est <= 0x7f800000u - 16u)) return false;  // also false for a NaN estimate
    const uint32_t below = s.codes & 0xffu, above = (s.codes >> 8) & 0xffu;
    bool upper[10];
    for (int j = 0; j < 10; ++j) upper[j] = x_to_bits(x_from_bits(est - 5 + (uint32_t)j) / ap) >= s.boundary;
    if (upper[0] || !upper[9]) return false;
    int at = 9;  // first j on the upper side
    for (int j = 8; j >= 1; --j) at = upper[j] ? j : at;
    for (int j = 1; j < 10; ++j)
        if (upper[j] != (j >= at)) return false;  // cannot happen with a monotone quotient; checked all the same
    const uint32_t found = est - 5 + (uint32_t)at;
    // quotient >= 0: the magnitude code; quotient < 0: with the sign bit, except 254
    const uint32_t below_minus = below == 254u ? 254u : (below | 0x80u), above_minus = above == 254u ? 254u : (above | 0x80u);
    const bool flip = precision < 0;  // then x >= 0 has the negative quotient
    *entry = flip ? XEntry{found, pack_codes(below_minus, above_minus, below, above)}
                  : XEntry{found, pack_codes(below, above, below_minus, above_minus)};
    return true;
}

// Entry of a bucket without a step: the codes below the step `step` (`above` false) or above it (`above` true).
CN_HD XEntry xlut_flat_entry(XEntry step, bool above) {
    const uint32_t c = step.codes;
    const uint32_t pos = above ? ((c >> 8) & 0xffu) : (c & 0xffu);
    const uint32_t neg = above ? ((c >> 24) & 0xffu) : ((c >> 16) & 0xffu);
    return XEntry{0xffffffffu, pack_codes(pos, pos, neg, neg)};
}

// Host: the steps of the precision-1 table, in ascending order.  A step can sit inside a bucket or
// exactly on its first pattern (then neither neighbour bucket shows two codes).  Returns their
// number, or -1 if the table is unusable or the codes do not run from 254 up to 127.
inline int xlut_collect_steps(const float *slot, XStep *out) {
    int count = 0;
    uint32_t current = 254u;  // code below the first bucket
    for (int i = 1; i < kXEntries - 1; ++i) {
        bool bad = false;
        const XEntry e = xlut_entry(i, 1.0f, slot, &bad);
        if (bad) return -1;
        const uint32_t below = magnitude_code(e.codes & 0xffu), above = magnitude_code((e.codes >> 8) & 0xffu);
        const uint32_t lo = (xlut_first(1.0f) + (uint32_t)(i - 1)) << kXShift;
        if (below != current) {
            if (count == kXMaxSteps) return -1;
            out[count++] = XStep{lo, current | (below << 8)};
        }
        if (above != below) {
            if (count == kXMaxSteps) return -1;
            out[count++] = XStep{e.boundary, below | (above << 8)};
        }
        current = above;
    }
    return current == 127u ? count : -1;
}

// Host: the whole table for `precision` from the steps, the way a workgroup builds it.  Returns
// false when the table must not be trusted.
inline bool xlut_build_from_steps(const XStep *steps, int count, float precision, const float *slot, XEntry *lut) {
    const uint32_t first = xlut_first(precision);
    bool bad = false, unusable = false;
    lut[0] = xlut_entry(0, precision, slot, &bad);
    unusable |= bad;
    lut[kXEntries - 1] = xlut_entry(kXEntries - 1, precision, slot, &bad);
    unusable |= bad;
    if ((uint64_t)first + kXBuckets > 0xff00u) unusable = true;  // infinity / NaN inside the window
    // a bucket without a step carries the codes above the nearest step below it; below the first step,
    // the codes below that one
    int previous = 0;
    XEntry e{}, before{};
    for (int k = 0; k < count && !unusable; ++k) {
        before = e;
        if (!xlut_locate_step(steps[k], precision, slot, &e)) { unusable = true; break; }
        const int64_t index = (int64_t)(e.boundary >> kXShift) - (int64_t)first + 1;
        if (index <= previous || index > kXBuckets) { unusable = true; break; }
        for (int i = previous + 1; i < index; ++i) lut[i] = k == 0 ? xlut_flat_entry(e, false) : xlut_flat_entry(before, true);
        lut[index] = e;
        previous = (int)index;
    }
    if (unusable || count == 0) return false;
    for (int i = previous + 1; i <= kXBuckets; ++i) lut[i] = xlut_flat_entry(e, true);
    return true;
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

// ---- the table on the quotient -------------------------------------------------------------------
// The literal procedure looks at x only through a = fl(x / precision), so its code is one fixed step function of
// the bit pattern of a, whatever the precision: the table above for precision 1 (where a = x) is that function.
// An encoder can therefore keep that one table and pay for the quotient per element instead of building a table
// per precision.  The quotient is formed as (float)((double)x * (1.0 / (double)precision)), which rounds the way
// x / precision does for every pair of fp32 operands whose quotient lies in the normal range: the product carries
// a relative error below 2^-51, and a quotient of two 24-bit significands is either representable or at least
// 2^-49 (relative) away from the nearest rounding boundary of the format, so the conversion falls on the same side;
// zeros, infinities and NaNs come out as the division's own (0 * inf = NaN = 0 / 0 and so on; a NaN's sign and
// payload do not matter to the code); no intermediate leaves the range of a double.  Below the normal range the
// two may differ in the last place, where every quotient has the code 254.
CN_HD double xlut_quotient_scale(float precision) { return 1.0 / (double)precision; }

CN_HD uint32_t xlut_code_by_quotient(uint32_t x_bits, double scale, const XEntry *table_of_one, uint32_t first_of_one) {
    const uint32_t a = x_to_bits((float)((double)x_from_bits(x_bits) * scale));
    return xlut_code(a, table_of_one[xlut_index(a & 0x7fffffffu, first_of_one)]);
}

}  // namespace cn
