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
// The build is what a call on a small input costs (about 4 us of the 7 us that a call on 4096 elements takes
// at the clocks such calls run at), so its phases keep their LDS reads independent of one another and the
// two sentinel entries, which take full evaluations of the literal procedure, are computed by lanes of
// wavefronts that locate no step.

struct EncodeShared {
    XEntry lut[kXEntries];
    float slot[128];
    int step_index[kXMaxSteps];
    XEntry step_entry[kXMaxSteps];
    uint8_t mark[(kXEntries + 3) / 4 * 4];  // 1 + number of the step that sits in this entry's bucket, 0 if none
};
static_assert(kXMaxSteps < 255, "a step's number plus one fits a byte");

// Returns true when the table in sh.lut may be used.
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
    __syncthreads();
    const uint32_t first = xlut_first(precision);
    bool bad = false;
    XEntry e{};
    int index = 0;
    if (t < count) {
        bad = !xlut_locate_step(mine, precision, sh.slot, &e);
        index = (int)(e.boundary >> kXShift) - (int)first + 1;
        if (bad || index < 1 || index > kXBuckets) { bad = true; index = 0; }
        sh.step_index[t] = index;
        if (index > 0) sh.mark[index] = (uint8_t)(t + 1);
    } else if (t == kEncodeThreads / 2) {       // the two sentinels: lanes of wavefronts that locate no step,
        sh.lut[0] = xlut_entry(0, precision, sh.slot, &bad);
    } else if (t == 3 * kEncodeThreads / 4) {   // so that they run beside the steps and not after them

        sh.lut[kXEntries - 1] = xlut_entry(kXEntries - 1, precision, sh.slot, &bad);
        if ((uint64_t)first + kXBuckets > 0xff00u) bad = true;  // infinity / NaN inside the window
    }
    if (t < count) sh.step_entry[t] = e;
    if (__syncthreads_or(bad ? 1 : 0)) return false;
    // the steps must come in ascending buckets, one per bucket
    bad = (t > 0 && t < count) ? (index <= sh.step_index[t - 1]) : false;
    if (__syncthreads_or(bad ? 1 : 0)) return false;
    // Every thread fills a run of consecutive entries.  An entry whose bucket holds a step is that step's
    // entry; any other carries the codes above the nearest step below it (below the first step: the codes
    // below that one).  Which step that is comes from the marks the locating threads left, so the table reads
    // of a run do not depend on one another.  The run length is odd: the lanes' 8-byte stores are then 2 (mod
    // 4) words apart and spread over all banks.
    constexpr int kRun = ((kXBuckets + kEncodeThreads - 1) / kEncodeThreads) | 1;
    const int i0 = 1 + t * kRun;
    // steps whose bucket lies before entry i0: a count over every sixteenth step, then over the sixteen behind
    // the last of those that qualify (two rounds of independent reads instead of a chain of eight)
    static_assert(kXMaxSteps % 16 == 0, "coarse stride");
    int coarse = 0;
#pragma unroll
    for (int c = 16; c <= kXMaxSteps; c += 16) coarse += (c <= count && sh.step_index[c - 1] < i0) ? 1 : 0;
    int below = 16 * coarse;
    {
        int fine = 0;
#pragma unroll
        for (int f = 0; f < 15; ++f) {
            const int k = 16 * coarse + f;
            fine += (k < count && sh.step_index[k < kXMaxSteps ? k : kXMaxSteps - 1] < i0) ? 1 : 0;
        }
        below += fine;
    }
    // Entries past the last bucket are clamped to it: those lanes compute and store the last bucket's own
    // entry again, which keeps the loop free of branches.
    uint32_t marks[kRun];
#pragma unroll
    for (int m = 0; m < kRun; ++m) marks[m] = sh.mark[i0 + m <= kXBuckets ? i0 + m : kXBuckets];
    uint32_t nearest = (uint32_t)below;  // 1 + number of the nearest step at or below the entry, 0 if none
#pragma unroll
    for (int m = 0; m < kRun; ++m) {
        nearest = marks[m] ? marks[m] : nearest;
        const XEntry of_step = sh.step_entry[nearest ? nearest - 1 : 0];
        const XEntry flat = xlut_flat_entry(of_step, nearest != 0);
        XEntry e_m;
        e_m.boundary = marks[m] ? of_step.boundary : flat.boundary;
        e_m.codes = marks[m] ? of_step.codes : flat.codes;
        sh.lut[i0 + m <= kXBuckets ? i0 + m : kXBuckets] = e_m;
    }
    __syncthreads();
    return true;
}

}  // namespace cn
