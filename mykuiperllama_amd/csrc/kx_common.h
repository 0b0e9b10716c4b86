// Shared device helpers and host-side argument checks for the gfx950 kernels.
#ifndef KX_COMMON_H
#define KX_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kx_hip.h"

namespace kx {

constexpr int kWave = 64;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// Workspace layout: [kCounterBytes of arrival counters, one per 64-byte line][fp32 partial sums].
// Counters that share a line serialise at the memory side (~10 ns per atomic, measured), so
// every (column tile, activation tile) pair gets a line of its own.
constexpr size_t kCounterBytes = 65536;
constexpr int kMaxTiles = kCounterBytes / 64;

// nibble i of a packed word holds column 8j + kOrder[i]
__host__ __device__ constexpr int order_of(int i) {
    return i < 4 ? 2 * i : 2 * (i - 4) + 1;
}

__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}

// Round to nearest even; NaN stays a quiet NaN.
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return static_cast<uint16_t>((u >> 16) | 0x0040u);
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return static_cast<float>(v);
}

inline hipStream_t as_stream(void* s) {
    return static_cast<hipStream_t>(s);
}

inline int launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? KX_OK : static_cast<int>(e);
}

}  // namespace kx

#endif  // KX_COMMON_H
