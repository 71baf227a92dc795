// Host-side construction of the encoder's bucket table.
//
// compression_8bit in the reference (source/clusterKernels.cu:1163-1232) runs a 6-step search over
// the 126-entry table for every element.  The code it produces is a monotone step function of the
// scaled magnitude a = |x / precision|: 254 below float(1.5e-6), then 0, 1, ..., 125, and 127 above
// float(0.995703).  A step function of an fp32 value can be evaluated with one table lookup
// indexed by the leading bits of the value's bit pattern, provided every bucket contains at most
// one step.  This file evaluates the reference procedure on the host to find the steps and lays
// them out per bucket; the device kernel then needs one LDS read and one comparison per element.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "cn_internal.h"

namespace cn {

static const uint32_t kTableBits[126] = {
#include "cn_table.inc"
};

static inline float as_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t as_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

void host_table(float out[126]) {
    for (int i = 0; i < 126; ++i) out[i] = as_float(kTableBits[i]);
}

// Magnitude code of a >= 0 (not NaN).  Equivalent form of the reference search: the pivot always
// ends on the even slot q = 2 * (number of odd-indexed entries below a); the answer is q or its
// lower odd neighbour.  Slot 126, which the reference never initialises, is taken as 1.0f.
uint8_t host_encode_magnitude(float a) {
    if (a < 0.0000015f) return 254;
    if (a > 0.995703f) return 127;
    float slot[127];
    host_table(slot);
    slot[126] = 1.0f;
    int q = 0;
    for (int p = 1; p < 126; p += 2)
        if (a > slot[p]) q += 2;
    if (q == 0) return (fabsf(slot[0] - a) < (slot[1] - a)) ? 0 : 1;
    return ((slot[q] - a) < fabsf(slot[q - 1] - a)) ? (uint8_t)q : (uint8_t)(q - 1);
}

static inline int rank_of(uint8_t code) { return code == 254 ? -1 : (int)code; }

bool build_encode_lut(EncodeLut *lut) {
    const uint32_t first = as_bits(0.0000015f) >> kBucketShift;
    const uint32_t last = as_bits(0.995703f) >> kBucketShift;
    const uint32_t count = last - first + 2;  // + one entry for everything above `last`
    if (count > sizeof(lut->entry) / sizeof(lut->entry[0])) {
        set_error("encoder table: %u buckets exceed the static capacity", count);
        return false;
    }
    lut->first_bucket = first;
    lut->count = count;

    // Pass 1: the boundary owned by each bucket (pattern of the first value that takes the higher
    // code) and the codes on either side of it.  A step that falls exactly on a bucket's first
    // pattern belongs to that bucket.
    constexpr size_t kCap = sizeof(lut->entry) / sizeof(lut->entry[0]);
    static uint32_t own[kCap];
    static uint8_t below[kCap], above[kCap];
    uint8_t prev_end = host_encode_magnitude(as_float(first << kBucketShift));
    for (uint32_t i = 0; i < count; ++i) {
        uint32_t lo = (first + i) << kBucketShift;
        uint32_t hi = (i == count - 1) ? lo : lo + (1u << kBucketShift) - 1;
        uint8_t begin = host_encode_magnitude(as_float(lo));
        uint8_t end = host_encode_magnitude(as_float(hi));
        if (rank_of(begin) < rank_of(prev_end) || rank_of(end) < rank_of(begin)) {
            set_error("encoder table: code is not monotone around bucket %u", first + i);
            return false;
        }
        own[i] = kNoBoundary;
        below[i] = above[i] = begin;
        if (prev_end != begin && begin != end) {
            set_error("encoder table: bucket %u holds more than one boundary", first + i);
            return false;
        }
        if (prev_end != begin) {
            own[i] = lo;
            below[i] = prev_end;
            above[i] = begin;
        } else if (begin != end) {
            uint32_t a = lo, b = hi;  // enc(a) == begin, enc(b) != begin
            while (b - a > 1) {
                uint32_t mid = a + (b - a) / 2;
                if (host_encode_magnitude(as_float(mid)) == begin) a = mid; else b = mid;
            }
            if (host_encode_magnitude(as_float(b)) != end) {
                set_error("encoder table: bucket %u holds more than one boundary", first + i);
                return false;
            }
            own[i] = b;
            above[i] = end;
        }
        prev_end = end;
    }

    // Pass 2: the kernel indexes with an approximate quotient that may be up to kGuard patterns
    // away from the exact one, so a bucket must also know a boundary that sits within 2*kGuard of
    // its edges in a neighbouring bucket.
    for (uint32_t i = 0; i < count; ++i) {
        uint32_t lo = (first + i) << kBucketShift;
        uint32_t next_lo = lo + (1u << kBucketShift);
        int src = -1, needed = 0;
        if (own[i] != kNoBoundary) { src = (int)i; ++needed; }
        if (i > 0 && own[i - 1] != kNoBoundary && lo - own[i - 1] <= 2 * kGuard) { src = (int)i - 1; ++needed; }
        if (i + 1 < count && own[i + 1] != kNoBoundary && own[i + 1] - next_lo < 2 * kGuard) { src = (int)i + 1; ++needed; }
        if (needed > 1) {
            set_error("encoder table: bucket %u needs %d boundaries", first + i, needed);
            return false;
        }
        if (src < 0) {
            lut->entry[i].boundary_minus_guard = kNoBoundary - kGuard;
            lut->entry[i].codes = (uint32_t)below[i] | ((uint32_t)below[i] << 8);
        } else {
            lut->entry[i].boundary_minus_guard = own[src] - kGuard;
            lut->entry[i].codes = (uint32_t)below[src] | ((uint32_t)above[src] << 8);
        }
    }
    return true;
}

}  // namespace cn

// Exported for host-only tests (no GPU needed): evaluates the table exactly as the device kernel's
// fast path does for an already-computed quotient pattern; *near is set when the kernel would take
// its exact path instead.
extern "C" int cn_host_encode_lut_lookup(uint32_t magnitude_bits, int *near) {
    static cn::EncodeLut lut;
    static int state = 0;
    if (state == 0) state = cn::build_encode_lut(&lut) ? 1 : -1;
    if (state < 0) return -1;
    uint32_t b = magnitude_bits >> cn::kBucketShift;
    uint32_t lo = lut.first_bucket, hi = lut.first_bucket + lut.count - 1;
    b = b < lo ? lo : (b > hi ? hi : b);
    const cn::EncodeBucket &e = lut.entry[b - lo];
    int32_t d = (int32_t)(magnitude_bits - e.boundary_minus_guard);
    if (near) *near = ((uint32_t)d <= 2 * cn::kGuard) ? 1 : 0;
    return (d >= (int32_t)cn::kGuard) ? (int)((e.codes >> 8) & 0xff) : (int)(e.codes & 0xff);
}

extern "C" int cn_host_encode_magnitude(float a) { return cn::host_encode_magnitude(a); }

// Bulk form of cn_host_encode_lut_lookup for exhaustive host tests.
extern "C" int cn_host_encode_lut_lookup_many(const uint32_t *magnitude_bits, size_t n, uint8_t *codes,
                                              uint8_t *near) {
    for (size_t i = 0; i < n; ++i) {
        int nr = 0;
        int c = cn_host_encode_lut_lookup(magnitude_bits[i], &nr);
        if (c < 0) return -1;
        codes[i] = (uint8_t)c;
        if (near) near[i] = (uint8_t)nr;
    }
    return 0;
}
