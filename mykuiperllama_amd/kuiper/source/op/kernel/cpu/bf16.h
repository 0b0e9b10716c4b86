// bf16 <-> fp32 and fp16 -> fp32 on the host (round to nearest even; NaN stays a quiet NaN).
#ifndef KUIPER_KERNEL_CPU_BF16_H
#define KUIPER_KERNEL_CPU_BF16_H

#include <cstdint>
#include <cstring>

namespace kernel {

inline float bf16_to_float(uint16_t h) {
    uint32_t u = static_cast<uint32_t>(h) << 16;
    float f;
    std::memcpy(&f, &u, sizeof(f));
    return f;
}

inline uint16_t float_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, sizeof(u));
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return static_cast<uint16_t>((u >> 16) | 0x0040u);
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

// what a bf16 tensor would hold: the value after one rounding
inline float round_bf16(float f) { return bf16_to_float(float_to_bf16(f)); }

// IEEE binary16 bits to fp32 (exact)
inline float fp16_to_float(uint16_t h) {
    const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
    const uint32_t exponent = (h >> 10) & 0x1fu;
    const uint32_t mantissa = h & 0x3ffu;
    uint32_t u;
    if (exponent == 0) {
        const float v = static_cast<float>(mantissa) * (1.0f / 16777216.0f);  // mantissa * 2^-24
        std::memcpy(&u, &v, sizeof(u));
        u |= sign;
    } else if (exponent == 31) {
        u = sign | 0x7f800000u | (mantissa << 13);
    } else {
        u = sign | ((exponent + 112u) << 23) | (mantissa << 13);
    }
    float f;
    std::memcpy(&f, &u, sizeof(f));
    return f;
}

}  // namespace kernel

#endif  // KUIPER_KERNEL_CPU_BF16_H
