// The encoder table of compression_8bit in LDS (device code only): shared by the codec kernel and by
// the kernels that encode a value they have just computed.
#pragma once

#include "cn_internal.h"
#include "cn_xlut.h"

namespace cn {

constexpr int kEncodeThreads = 256;  // threads that build the table; a workgroup may have more

// ---- encoder ---------------------------------------------------------------------------------------
// Every workgroup builds the table of cn_xlut.h for the call's precision in LDS (one thread per step
// of the code function: nine evaluations of the literal procedure and a run of LDS stores), then
// looks every element up: shift, clamp, one 8-byte LDS read, one compare, one byte select.

struct EncodeShared {
    XEntry lut[kXEntries];
    float slot[128];
    int step_index[kXMaxSteps];
    XEntry step_entry[kXMaxSteps];
};

// Returns true when the table in sh.lut may be used.
__device__ __forceinline__ bool build_table(EncodeShared &sh, const XStep *__restrict__ steps, int count,
                                            float precision, const float *__restrict__ table) {
    const int t = threadIdx.x;
    if (t < 126) sh.slot[t] = table[t];
    if (t == 126) sh.slot[126] = 1.0f;
    if (t == 127) sh.slot[127] = 0.0f;
    __syncthreads();
    const uint32_t first = xlut_first(precision);
    bool bad = false;
    XEntry e{};
    int index = 0;
    if (t < count) {
        bad = !xlut_locate_step(steps[t], precision, sh.slot, &e);
        index = (int)(e.boundary >> kXShift) - (int)first + 1;
        if (bad || index < 1 || index > kXBuckets) { bad = true; index = 0; }
        sh.step_index[t] = index;
    } else if (t == count) {
        sh.lut[0] = xlut_entry(0, precision, sh.slot, &bad);
    } else if (t == count + 1) {
        sh.lut[kXEntries - 1] = xlut_entry(kXEntries - 1, precision, sh.slot, &bad);
        if ((uint64_t)first + kXBuckets > 0xff00u) bad = true;  // infinity / NaN inside the window
    }
    if (t < count) sh.step_entry[t] = e;
    if (__syncthreads_or(bad ? 1 : 0)) return false;
    // the steps must come in ascending buckets, one per bucket
    bad = (t > 0 && t < count) ? (index <= sh.step_index[t - 1]) : false;
    if (__syncthreads_or(bad ? 1 : 0)) return false;
    // Every thread fills a run of consecutive entries: the step whose bucket it is, else the codes
    // below the next step (above the last one).
    constexpr int kRun = (kXBuckets + kEncodeThreads - 1) / kEncodeThreads;
    const int i0 = 1 + t * kRun;
    const int i1 = (i0 + kRun < kXBuckets + 1) ? i0 + kRun : kXBuckets + 1;
    int k = 0;  // first step at or above entry i0
    for (int width = 128; width > 0; width >>= 1)
        if (k + width <= count && sh.step_index[k + width - 1] < i0) k += width;
    int next_index = k < count ? sh.step_index[k] : 0x7fffffff;
    XEntry next_entry = sh.step_entry[k < count ? k : count - 1];
    for (int i = i0; i < i1; ++i) {
        if (i == next_index) {
            sh.lut[i] = next_entry;
            ++k;
            next_index = k < count ? sh.step_index[k] : 0x7fffffff;
            if (k < count) next_entry = sh.step_entry[k];
            continue;
        }
        sh.lut[i] = xlut_flat_entry(next_entry, k >= count);
    }
    __syncthreads();
    return true;
}

}  // namespace cn
