// Host build of the encoder table (cn_xlut.h) for the CPU tests: the same inline functions the
// device kernels use, evaluated on the host, so that table construction and lookup can be checked
// exhaustively against the CPU checker without a GPU.  Nothing on the device path calls this file.
#include <vector>

#include "cn_internal.h"
#include "cn_xlut.h"

namespace cn {

static const uint32_t kTableBits[126] = {
#include "cn_table.inc"
};

// The 126-entry codebook, exact bit patterns of the reference's table file.
void host_table(float out[126]) {
    for (int i = 0; i < 126; ++i) out[i] = x_from_bits(kTableBits[i]);
}

}  // namespace cn

namespace {

void host_slot(float slot[128]) {
    cn::host_table(slot);
    slot[126] = 1.0f;
    slot[127] = 0.0f;
}

}  // namespace

extern "C" {

int cn_host_xlut_entries(void) { return cn::kXEntries; }

int cn_host_xlut_step_count(void) {
    float slot[128];
    host_slot(slot);
    static cn::XStep steps[cn::kXMaxSteps];
    return cn::xlut_collect_steps(slot, steps);
}

// Fills entries[kXEntries] (8 bytes each: boundary, codes) and *first for `precision`, from the list
// of steps, the way a workgroup of the encoder does; returns 1 if
// the table must not be trusted for this precision (the encoder then evaluates every element
// literally), else 0.
int cn_host_xlut_build(float precision, void *entries, uint32_t *first) {
    float slot[128];
    host_slot(slot);
    static cn::XStep steps[cn::kXMaxSteps];
    static int count = -2;
    if (count == -2) count = cn::xlut_collect_steps(slot, steps);
    if (first) *first = cn::xlut_first(precision);
    if (count <= 0) return 1;
    return cn::xlut_build_from_steps(steps, count, precision, slot, static_cast<cn::XEntry *>(entries)) ? 0 : 1;
}

// The encoder as the device runs it: table lookup, or the literal procedure when the table is
// reported unusable.  Returns which of the two was used (1 = table).
int cn_host_xlut_encode_many(float precision, const float *x, size_t n, uint8_t *codes) {
    float slot[128];
    host_slot(slot);
    std::vector<cn::XEntry> lut(cn::kXEntries);
    uint32_t first = 0;
    const int unusable = cn_host_xlut_build(precision, lut.data(), &first);
    for (size_t i = 0; i < n; ++i) {
        if (unusable) {
            codes[i] = (uint8_t)cn::encode_exact(x[i], precision, slot);
        } else {
            const uint32_t bits = cn::x_to_bits(x[i]);
            codes[i] = (uint8_t)cn::xlut_code(bits, lut[cn::xlut_index(bits & 0x7fffffffu, first)]);
        }
    }
    return unusable ? 0 : 1;
}

// The encoder on the quotient as the device runs it: the table for precision 1 and the quotient formed as a
// product in double precision.  Returns 1, or 0 if the table for precision 1 cannot be built.
int cn_host_quotient_encode_many(float precision, const float *x, size_t n, uint8_t *codes) {
    static std::vector<cn::XEntry> of_one;
    static int usable = -1;
    if (usable < 0) {
        of_one.resize(cn::kXEntries);
        uint32_t first = 0;
        usable = cn_host_xlut_build(1.0f, of_one.data(), &first) == 0 ? 1 : 0;
    }
    if (!usable) return 0;
    const uint32_t first_of_one = cn::xlut_first(1.0f);
    const double scale = cn::xlut_quotient_scale(precision);
    for (size_t i = 0; i < n; ++i)
        codes[i] = (uint8_t)cn::xlut_code_by_quotient(cn::x_to_bits(x[i]), scale, of_one.data(), first_of_one);
    return 1;
}

int cn_host_encode_exact(float x, float precision) {
    float slot[128];
    host_slot(slot);
    return (int)cn::encode_exact(x, precision, slot);
}

}  // extern "C"
