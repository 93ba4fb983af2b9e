/*
 * selfcheck.c — sweeps that pin the oracle's f32->f16 narrowing against the
 * CPU's own F16C conversion (vcvtps2ph, round-to-nearest-even), an independent
 * implementation of the same IEEE operation.  Test infrastructure only.
 */
#include <immintrin.h>
#include <stdint.h>
#include <string.h>

uint16_t lq4o_f32_to_f16(float v);

/* Compares every `stride`-th f32 bit pattern in [first, last] (NaNs skipped:
 * their payload rule is a convention, checked separately).  Returns the number
 * of mismatches and stores the first offending pattern. */
uint64_t lq4o_sweep_f32_to_f16_vs_f16c(uint32_t first, uint32_t last, uint32_t stride,
                                       uint32_t* first_bad) {
    uint64_t bad = 0;
    uint64_t b = first;
    for (; b <= (uint64_t)last; b += stride) {
        uint32_t bits = (uint32_t)b;
        if ((bits & 0x7f800000u) == 0x7f800000u && (bits & 0x007fffffu)) continue;
        float f;
        memcpy(&f, &bits, 4);
        uint16_t hw = (uint16_t)_mm_extract_epi16(
            _mm_cvtps_ph(_mm_set_ss(f), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC), 0);
        if (hw != lq4o_f32_to_f16(f)) {
            if (!bad && first_bad) *first_bad = bits;
            ++bad;
        }
    }
    return bad;
}
