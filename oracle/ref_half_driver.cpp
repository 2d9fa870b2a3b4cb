// Thin C wrapper around the reference's own fp16 <-> fp32 routines, compiled from the reference
// header where it lies (include/ppml/HalfUtils.h:26-52).  TEST INFRASTRUCTURE ONLY: it exists
// so the oracle's fp16 conversion can be checked against the real reference code.
// No reference source is copied; the header is included by path at build time.
#include <cstdint>
#include "ppml/HalfUtils.h"

extern "C" uint16_t ref_fp32_to_fp16(float f) { return ppml::fp32_to_fp16(f); }
extern "C" float ref_fp16_to_fp32(uint16_t h) { return ppml::fp16_to_fp32(h); }

// Sweeps every `stride`-th binary32 bit pattern starting at `start` and returns the number of
// patterns on which `fn` (the oracle's conversion) disagrees with the reference's.
extern "C" int64_t ref_sweep_fp32_to_fp16(uint16_t (*fn)(float), uint32_t start, uint32_t stride,
                                          uint32_t *first_bad) {
    int64_t bad = 0;
    uint64_t u = start;
    for (; u <= 0xffffffffull; u += stride) {
        const float f = ppml::fp32_from_bits(static_cast<uint32_t>(u));
        if (fn(f) != ppml::fp32_to_fp16(f)) {
            if (!bad && first_bad) *first_bad = static_cast<uint32_t>(u);
            ++bad;
        }
    }
    return bad;
}
