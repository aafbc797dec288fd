/*
 * f16c_check.c -- pins the oracle's software fp32->fp16 converter against the
 * CPU's F16C hardware converter (VCVTPS2PH, round-to-nearest-even), which is an
 * independent implementation of the same IEEE conversion that __float2half
 * (src/OperationKernels.cu:854 of the reference) performs.
 * TEST INFRASTRUCTURE ONLY.
 */
#include <immintrin.h>
#include <stdint.h>
#include <string.h>
#include "nz_oracle.h"

/* Hardware conversion of one value (bits in, bits out). */
uint16_t nzo_f16c_hw_bits(uint32_t fbits) {
    float f;
    memcpy(&f, &fbits, 4);
    return (uint16_t)_cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
}

/* Compare software vs hardware over fp32 bit patterns start, start+step, ...
 * (count of them). Returns the number of mismatches; *first_bad receives the
 * first mismatching pattern. NaNs must agree bit-for-bit as well. */
uint64_t nzo_f16c_compare_range(uint64_t start, uint64_t count, uint64_t step, uint32_t* first_bad) {
    uint64_t bad = 0;
    uint32_t fb = 0;
    int have = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad)
    for (uint64_t i = 0; i < count; i++) {
        const uint32_t u = (uint32_t)(start + i * step);
        float f;
        memcpy(&f, &u, 4);
        const uint16_t sw = nzo_f32_to_f16_bits(f);
        const uint16_t hw = (uint16_t)_cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
        if (sw != hw) {
            bad++;
#pragma omp critical
            if (!have || u < fb) { fb = u; have = 1; }
        }
    }
    if (first_bad) *first_bad = fb;
    return bad;
}

/* Round trip of every half through the widening converter vs hardware VCVTPH2PS. */
uint32_t nzo_f16c_compare_widen(void) {
    uint32_t bad = 0;
    for (uint32_t h = 0; h < 65536; h++) {
        const float sw = nzo_f16_bits_to_f32((uint16_t)h);
        const float hw = _cvtsh_ss((uint16_t)h);
        uint32_t a, b;
        memcpy(&a, &sw, 4);
        memcpy(&b, &hw, 4);
        if (a != b) bad++;
    }
    return bad;
}
