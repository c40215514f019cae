// fp32 -> bf16 narrowing as the reference's bfloat16_t assignment does it (include/bfloat16.h:40-65):
// round to nearest even on normals, subnormals flushed to signed zero, infinities kept, NaN quieted.
// Pure integer arithmetic on the bit pattern, so the same text compiles for the device and for a
// host-side exhaustive check of all 2^32 inputs.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define XFT_HOST_DEVICE __host__ __device__
#else
#define XFT_HOST_DEVICE
#endif

namespace xfthip {

XFT_HOST_DEVICE inline uint16_t f32_bits_to_bf16_ref(uint32_t u) {
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    if (a == 0x7F800000u) return (uint16_t)(u >> 16);
    if (a < 0x00800000u) return (uint16_t)((u >> 16) & 0x8000u);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

// The same function without early returns: selects instead of a branch ladder, so that the eight
// conversions of an output chunk stay straight-line code.
XFT_HOST_DEVICE inline uint32_t f32_bits_to_bf16_sel(uint32_t u) {
    const uint32_t a = u & 0x7FFFFFFFu, top = u >> 16;
    uint32_t r = (u + 0x7FFFu + (top & 1u)) >> 16;
    r = a < 0x00800000u ? (top & 0x8000u) : r;
    r = a >= 0x7F800000u ? (top | (a > 0x7F800000u ? 0x40u : 0u)) : r;
    return r;
}

} // namespace xfthip
