// bf16 <-> fp32 on the host (round to nearest even; NaN stays a quiet NaN).
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

}  // namespace kernel

#endif  // KUIPER_KERNEL_CPU_BF16_H
