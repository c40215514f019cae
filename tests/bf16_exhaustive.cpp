// Host-side exhaustive check of the library's two fp32 -> bf16 narrowing functions
// (xfastertransformer_amd/csrc/bf16_convert.h, the text the device kernels compile) against the
// oracle's restatement of the reference conversion, over all 2^32 bit patterns.
// Built and run by tests/test_oracle_pins.py; prints the number of mismatches.
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "bf16_convert.h"

extern "C" uint16_t orc_f32_to_bf16(float f);

int main() {
    unsigned long long bad_ref = 0, bad_sel = 0;
#pragma omp parallel for reduction(+ : bad_ref, bad_sel) schedule(static)
    for (long long i = 0; i < (1LL << 32); ++i) {
        const uint32_t u = (uint32_t)i;
        float f;
        memcpy(&f, &u, 4);
        const uint16_t want = orc_f32_to_bf16(f);
        bad_ref += xfthip::f32_bits_to_bf16_ref(u) != want;
        bad_sel += (uint16_t)xfthip::f32_bits_to_bf16_sel(u) != want || (xfthip::f32_bits_to_bf16_sel(u) >> 16) != 0;
    }
    printf("mismatches ref=%llu sel=%llu\n", bad_ref, bad_sel);
    return (bad_ref || bad_sel) ? 1 : 0;
}
