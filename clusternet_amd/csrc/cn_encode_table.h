// The encoder table of compression_8bit in LDS (device code only): shared by the codec kernel and by
// the kernels that encode a value they have just computed.
#pragma once

#include "cn_internal.h"
#include "cn_xlut.h"

namespace cn {

constexpr int kEncodeThreads = 256;  // threads that build the table; a workgroup may have more

// ---- encoder ---------------------------------------------------------------------------------------
// Every workgroup builds the table of cn_xlut.h for the call's precision in LDS (one thread per step
// of the code function: ten divisions around the step's estimated position; then every thread a run of
// LDS stores), then looks every element up: shift, clamp, one 8-byte LDS read, one compare, one byte select.
// The build is what a call on a small input costs (about 3.6 us of the 7 us that a call on 4096 elements
// takes), so its phases keep their LDS reads independent of one another and the
// two sentinel entries, which take full evaluations of the literal procedure, are computed by lanes of
// wavefronts that locate no step.

struct EncodeShared {
    XEntry lut[kXEntries];
    float slot[128];
    int step_index[kXMaxSteps];
    XEntry step_entry[kXMaxSteps];
    uint8_t mark[(kXEntries + 3) / 4 * 4];  // 1 + number of the step that sits in this entry's bucket, 0 if none
    uint32_t sentinel_code[8];              // literal codes at the eight patterns that define the two sentinel entries
};
static_assert(kXMaxSteps < 255, "a step's number plus one fits a byte");

// Returns true when the table in sh.lut may be used.
//
// The build is a chain of latencies (a workgroup of a small call does little else), so it is laid out for a short
// critical path: a thread's own step comes from global memory together with the codebook and is located in
// registers before the first barrier; the eight literal evaluations behind the two sentinel entries run one per
// lane on wavefronts that locate no step; every group of LDS reads is issued as a whole before its first use
// (unconditional loads, conditions applied to the values), because a conditional read costs a full LDS round
// trip each.  Measured at the shader clock: about 9 000 cycles, against 11 000 with dependent reads.
__device__ __forceinline__ bool build_table(EncodeShared &sh, const XStep *__restrict__ steps, int count,
                                            float precision, const float *__restrict__ table) {
    const int t = threadIdx.x;
    // requested together with the table value (and with the precision, if the caller reads it from memory):
    // one memory latency in front of the table instead of three
    const XStep mine = steps[t < count ? t : 0];
    for (int w = t; w < (int)(sizeof(sh.mark) / 4); w += kEncodeThreads) reinterpret_cast<uint32_t *>(sh.mark)[w] = 0u;
    if (t < 126) sh.slot[t] = table[t];
    if (t == 126) sh.slot[126] = 1.0f;
    if (t == 127) sh.slot[127] = 0.0f;
    const uint32_t first = xlut_first(precision);
    // the own step: registers only, needs nothing of the above
    bool bad = false;
    XEntry e{};
    int index = 0;
    if (t < count) {
        bad = !xlut_locate_step(mine, precision, nullptr, &e);
        index = (int)(e.boundary >> kXShift) - (int)first + 1;
        if (bad || index < 1 || index > kXBuckets) { bad = true; index = 0; }
    }
    __syncthreads();  // the codebook copy and the cleared marks are there
    if (t < count) {
        sh.step_index[t] = index;
        sh.step_entry[t] = e;
        if (index > 0) sh.mark[index] = (uint8_t)(t + 1);
    }
    // The sentinels (xlut_entry for the entries 0 and kXEntries - 1) take literal evaluations at eight patterns:
    // lane j of the third wavefront evaluates pattern j, one lane assembles the two entries behind the barrier.
    const uint32_t kSign = 0x80000000u;
    const uint32_t top = first > 0 ? (first << kXShift) - 1 : 0u;
    const uint64_t start64 = ((uint64_t)first + kXBuckets) << kXShift;
    const uint32_t start = start64 > 0x7f800000u ? 0x7f800000u : (uint32_t)start64;
    constexpr int kSentinelLane = kEncodeThreads / 2;
    if (t >= kSentinelLane && t < kSentinelLane + 8) {
        const uint32_t pattern[8] = {top, top | kSign, 0x7fc00000u, 0xffc00000u, start, start | kSign, 0x7f800000u, 0xff800000u};
        uint32_t mine_bits = pattern[0];
#pragma unroll
        for (int j = 1; j < 8; ++j) mine_bits = (t - kSentinelLane == j) ? pattern[j] : mine_bits;
        sh.sentinel_code[t - kSentinelLane] = encode_exact(x_from_bits(mine_bits), precision, sh.slot);
    }
    __syncthreads();
    // the steps must come in ascending buckets, one per bucket
    if (t > 0 && t < count) bad = bad || (index <= sh.step_index[t - 1]);
    if (t == kSentinelLane) {
        uint32_t c[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) c[j] = sh.sentinel_code[j];
        // entry 0: everything below bucket `first` must be code 254, up to its largest pattern
        if (first > 0 && (c[0] != 254u || c[1] != 254u)) bad = true;
        sh.lut[0] = XEntry{0xffffffffu, pack_codes(254, 254, 254, 254)};
        // last entry: one code from the end of the last bucket up to infinity, then the code of a NaN
        XEntry last;
        if (start64 > 0x7f800000u) {
            last = XEntry{0u, pack_codes(c[2], c[2], c[3], c[3])};  // only NaNs left
        } else {
            if (c[4] != c[6] || c[5] != c[7]) bad = true;
            last = XEntry{0x7f800001u, pack_codes(c[4], c[2], c[5], c[3])};
        }
        sh.lut[kXEntries - 1] = last;
        if ((uint64_t)first + kXBuckets > 0xff00u) bad = true;  // infinity / NaN inside the window
    }
    if (__syncthreads_or(bad ? 1 : 0)) return false;
    // Every thread fills a run of consecutive entries.  An entry whose bucket holds a step is that step's
    // entry; any other carries the codes above the nearest step below it (below the first step: the codes
    // below that one).  Which step that is comes from the marks the locating threads left, so the table reads
    // of a run do not depend on one another.  The run length is odd: the lanes' 8-byte stores are then 2 (mod
    // 4) words apart and spread over all banks.
    constexpr int kRun = ((kXBuckets + kEncodeThreads - 1) / kEncodeThreads) | 1;
    const int i0 = 1 + t * kRun;
    // steps whose bucket lies before entry i0: a count over every sixteenth step, then over the fifteen behind
    // the last of those that qualify: two rounds of independent reads
    static_assert(kXMaxSteps % 16 == 0, "coarse stride");
    int every16th[kXMaxSteps / 16];
#pragma unroll
    for (int c = 0; c < kXMaxSteps / 16; ++c) every16th[c] = sh.step_index[16 * c + 15];
    int coarse = 0;
#pragma unroll
    for (int c = 0; c < kXMaxSteps / 16; ++c) coarse += ((16 * c + 16 <= count) & (every16th[c] < i0)) ? 1 : 0;
    int behind[15];
#pragma unroll
    for (int f = 0; f < 15; ++f) {
        const int k = 16 * coarse + f;
        behind[f] = sh.step_index[k < kXMaxSteps ? k : kXMaxSteps - 1];
    }
    int below = 16 * coarse;
#pragma unroll
    for (int f = 0; f < 15; ++f) below += ((16 * coarse + f < count) & (behind[f] < i0)) ? 1 : 0;
    // Entries past the last bucket are clamped to it: those lanes compute and store the last bucket's own
    // entry again, which keeps the loop free of branches.
    uint32_t marks[kRun];
#pragma unroll
    for (int m = 0; m < kRun; ++m) marks[m] = sh.mark[i0 + m <= kXBuckets ? i0 + m : kXBuckets];
    uint32_t nearest[kRun];  // 1 + number of the nearest step at or below the entry, 0 if none
    uint32_t running = (uint32_t)below;
#pragma unroll
    for (int m = 0; m < kRun; ++m) {
        running = marks[m] ? marks[m] : running;
        nearest[m] = running;
    }
    XEntry of_step[kRun];
#pragma unroll
    for (int m = 0; m < kRun; ++m) of_step[m] = sh.step_entry[nearest[m] ? nearest[m] - 1 : 0];
#pragma unroll
    for (int m = 0; m < kRun; ++m) {
        const XEntry flat = xlut_flat_entry(of_step[m], nearest[m] != 0);
        XEntry e_m;
        e_m.boundary = marks[m] ? of_step[m].boundary : flat.boundary;
        e_m.codes = marks[m] ? of_step[m].codes : flat.codes;
        sh.lut[i0 + m <= kXBuckets ? i0 + m : kXBuckets] = e_m;
    }
    __syncthreads();
    return true;
}

// ---- the encoder on the quotient ---------------------------------------------------------------------
// The table of cn_xlut.h for precision 1 is the code as a function of the quotient x / precision (see there); it is
// built and verified once on the host at initialisation and kept in device memory.  A workgroup copies it into LDS
// (kXEntries entries of 8 bytes) instead of building a table for the call's precision, and pays three instructions
// per element for the quotient (conversion, fp64 product, conversion).
constexpr int kQuotientTableVecs = kXEntries * (int)sizeof(XEntry) / 16;
static_assert(kXEntries * sizeof(XEntry) % 16 == 0, "whole 16-byte vectors");

typedef uint32_t qt_u32x4 __attribute__((ext_vector_type(4)));

// Requests this thread's share of the table; `store_quotient_table` puts it into LDS.  Split so that the caller can issue
// other loads in between; a barrier must follow the store.
template <int kThreadsOfGroup>
struct QuotientTableCopy {
    static constexpr int kEach = (kQuotientTableVecs + kThreadsOfGroup - 1) / kThreadsOfGroup;
    qt_u32x4 part[kEach];
    __device__ __forceinline__ void request(const XEntry *__restrict__ table_in_memory) {
        const qt_u32x4 *src = reinterpret_cast<const qt_u32x4 *>(table_in_memory);
#pragma unroll
        for (int j = 0; j < kEach; ++j) {
            const int at = j * kThreadsOfGroup + (int)threadIdx.x;
            part[j] = src[at < kQuotientTableVecs ? at : kQuotientTableVecs - 1];
        }
    }
    __device__ __forceinline__ void store(XEntry *lut) {
        qt_u32x4 *dst = reinterpret_cast<qt_u32x4 *>(lut);
#pragma unroll
        for (int j = 0; j < kEach; ++j) {
            const int at = j * kThreadsOfGroup + (int)threadIdx.x;
            if (at < kQuotientTableVecs) dst[at] = part[j];
        }
    }
};

__device__ __forceinline__ double quotient_scale(float precision) { return xlut_quotient_scale(precision); }

__device__ __forceinline__ uint32_t encode_by_quotient(uint32_t x_bits, double scale, const XEntry *lut, uint32_t first_of_one) {
    return xlut_code_by_quotient(x_bits, scale, lut, first_of_one);
}

}  // namespace cn
