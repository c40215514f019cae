// Helpers shared by the host-side sources (xft_layers.cpp, xft_models.cpp): error handling in the
// reference's style (print and exit), one-time device initialisation, 16-bit float conversions
// and the fp32 -> device-weight conversion.  Plain C++, no HIP headers.
#pragma once
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

#include "../../../include/dtype.h"
#include "../../../include/xft_hip.h"

namespace xfthost {

[[noreturn]] inline void die(const char *what) {
    printf("%s: %s\n", what, xfthip_last_error());
    exit(-1);
}

#define CK(call)                   \
    do {                           \
        if ((call) != 0) die(#call); \
    } while (0)

inline void ensure_init() {
    static std::once_flag once;
    std::call_once(once, [] {
        int dev = 0;
        if (const char *e = getenv("XFT_HIP_DEVICE")) dev = atoi(e);
        CK(xfthip_init(dev));
    });
}

// fp32 -> bf16 as the reference's bfloat16_t does (include/bfloat16.h:40-65)
inline uint16_t to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    if (a == 0x7F800000u) return (uint16_t)(u >> 16);
    if (a < 0x00800000u) return (uint16_t)((u >> 16) & 0x8000u);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
inline float from_bf16(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

// weight kind for a DataType; -1 (after the reference's own message) for a type no entry point serves
inline int kind_of(xft::DataType dt) {
    switch (dt) {
        case xft::DataType::bf16: return XFTHIP_W_BF16;
        case xft::DataType::fp16: {
            static std::once_flag once;
            std::call_once(once, [] { printf(">> fp16 weights are held as bf16 by this build\n"); });
            return XFTHIP_W_BF16;
        }
        case xft::DataType::int8: return XFTHIP_W_INT8;
        case xft::DataType::w8a8: return XFTHIP_W_W8A8;
        case xft::DataType::int4: return XFTHIP_W_UINT4;
        case xft::DataType::nf4: return XFTHIP_W_NF4;
        default: printf(">> unsupported data type\n"); return -1;
    }
}

// Convert a contiguous fp32 [K, N] host matrix into a device weight handle of `kind`.
inline xfthip_weight_t make_weight(int kind, int K, int N, const float *W, int flags) {
    xfthip_weight_t h = nullptr;
    if (kind == XFTHIP_W_BF16) {
        std::vector<uint16_t> b((size_t)K * N);
        for (size_t i = 0; i < b.size(); ++i) b[i] = to_bf16(W[i]);
        CK(xfthip_weight_create(kind, K, N, b.data(), nullptr, nullptr, flags, &h));
        return h;
    }
    std::vector<float> scale(N), zero(N, 0.0f);
    std::vector<uint8_t> q((size_t)K * N);
    CK(xfthip_quantize_weight(kind, K, N, W, q.data(), scale.data(), zero.data()));
    CK(xfthip_weight_create(kind, K, N, q.data(), scale.data(), kind == XFTHIP_W_NF4 ? nullptr : zero.data(), flags, &h));
    return h;
}

// fp16 bit pattern -> float (IEEE binary16)
inline float from_fp16(uint16_t h) {
    const uint32_t sgn = (uint32_t)(h & 0x8000u) << 16, ex = (h >> 10) & 31u;
    uint32_t man = h & 1023u, u;
    if (ex == 0) {
        if (man == 0) {
            u = sgn;
        } else {
            int sh = 0;
            while (!(man & 1024u)) man <<= 1, ++sh;
            u = sgn | ((uint32_t)(113 - sh) << 23) | ((man & 1023u) << 13);
        }
    } else if (ex == 31) {
        u = sgn | 0x7F800000u | (man << 13);
    } else {
        u = sgn | ((ex + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}
// float -> fp16 bit pattern, round to nearest even
inline uint16_t to_fp16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint32_t sgn = (u >> 16) & 0x8000u, a = u & 0x7FFFFFFFu;
    if (a >= 0x47800000u) return (uint16_t)(sgn | (a > 0x7F800000u ? 0x7E00u : 0x7C00u));
    if (a < 0x38800000u) {
        if (a < 0x33000000u) return (uint16_t)sgn;
        const uint32_t man = (a & 0x7FFFFFu) | 0x800000u;
        const int sh = 126 - (int)(a >> 23);
        uint32_t r = man >> sh;
        const uint32_t rem = man & ((1u << sh) - 1), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (r & 1u))) ++r;
        return (uint16_t)(sgn | r);
    }
    const uint32_t r = a - 0x38000000u;
    uint32_t man = r >> 13;
    const uint32_t rem = r & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (man & 1u))) ++man;
    return (uint16_t)(sgn | man);
}

} // namespace xfthost
