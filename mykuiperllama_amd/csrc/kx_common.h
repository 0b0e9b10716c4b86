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

// Workspace layout: [kCounterBytes, zeroed once and left zeroed by every launch][fp32 partial sums].
// The zeroed area holds, depending on the launch, arrival counters on 64-byte lines of their own (counters that
// share a line serialise at the memory side, ~10 ns per atomic, measured; every (column tile, activation tile)
// pair gets four lines, one per quarter of the tile, for the exchange in which every wave of 64 columns reports
// for itself) or, for the fixed-point exchange of the one-row plain launch, a 64-bit slot and a 64-bit mask word
// per output column (up to 32 768 columns).
constexpr int kCountersPerTile = 4;
constexpr size_t kCounterBytes = 524288;
constexpr int kMaxTiles = kCounterBytes / 64 / kCountersPerTile;

// nibble i of a packed word holds column 8j + kOrder[i]
__host__ __device__ constexpr int order_of(int i) {
    return i < 4 ? 2 * i : 2 * (i - 4) + 1;
}

__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}

// Round to nearest even; NaN stays a quiet NaN, (bits >> 16) | 0x0040.  gfx950 converts in hardware
// (v_cvt_pk_bf16_f32); the instruction agrees with the integer formulation
//   u += 0x7fff + ((u >> 16) & 1); return u >> 16     (NaN handled apart as above)
// on every one of the 2^32 inputs.
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    const __bf16 b = static_cast<__bf16>(f);
    uint16_t out;
    __builtin_memcpy(&out, &b, 2);
    return out;
}

// two conversions in one instruction: lo in bits 0..15, hi in bits 16..31
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const bf16x2_t b = __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t);
    uint32_t out;
    __builtin_memcpy(&out, &b, 4);
    return out;
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return static_cast<float>(v);
}

// The results of a one-row launch leave with the device-scope bit: the store is written through the XCD's L2 to
// memory at once, so the end of the kernel finds no dirty lines to write back.  Measured on the one-row AWQ
// GEMV: 0.1-0.2 us per launch (1.9 % on the seven-projection step) against plain stores.  Not for bulk: the
// launches of a step with 8 or 16 sequences write enough for the write-through traffic to cost 1.5-4 % of the
// step, and 150 000 waves that each store two bytes of an lm_head row lose 8 us; those keep plain stores.
template <typename T>
__device__ __forceinline__ void store_result(T* p, T v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// bf16(silu(g)), g / (1 + exp(-g)), as every SwiGLU of the library computes it: the hardware's exponential and
// reciprocal (v_exp_f32, v_rcp_f32: each good to about one unit in the last place of fp32, the product
// -g * log2(e) to a few more for large |g|), far inside the bf16 rounding that follows.  The library expf and a
// true division cost some 35 instructions per element against 8, which a launch that produces sixteen rows of
// activations in its prologue feels (down projection at sixteen rows: 26.0 -> 23.5 us).
__device__ __forceinline__ float silu_rounded_to_bf16(float g) {
    const float e = __builtin_amdgcn_exp2f(-g * 1.44269504088896341f);
    return bf16_to_f32(f32_to_bf16(g * __builtin_amdgcn_rcpf(1.0f + e)));
}

// Operand and result types of v_mfma_f32_16x16x32_bf16: lane l supplies eight consecutive k
// (8*(l/16) .. +7) of row (A) or column (B) l%16 and receives D[4*(l/16)+v][l%16], v = 0..3.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 as_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    u32x4 v = {a, b, c, d};
    bf16x8 out;
    __builtin_memcpy(&out, &v, 16);
    return out;
}

// Lane exchanges inside a row of 16 lanes ride on the VALU's data-parallel-primitive operand path
// (one instruction for move + add), where a ds_bpermute costs an LDS round trip of ~100 cycles that a
// dependent chain cannot hide.  CTRL 0x120 + n rotates a row right by n lanes.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// every lane of a 16-lane row receives the row's sum (lanes may differ in the last bit: each adds
// the same sixteen numbers in its own rotated order)
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_move<0x128>(v);
    v += dpp_move<0x124>(v);
    v += dpp_move<0x122>(v);
    v += dpp_move<0x121>(v);
    return v;
}

__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_move<0x128>(v));
    v = fmaxf(v, dpp_move<0x124>(v));
    v = fmaxf(v, dpp_move<0x122>(v));
    v = fmaxf(v, dpp_move<0x121>(v));
    return v;
}

__device__ __forceinline__ float read_lane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// wave-wide reductions, the same value in every lane: rows by rotation, the four rows through
// scalar registers
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    return (read_lane(v, 0) + read_lane(v, 16)) + (read_lane(v, 32) + read_lane(v, 48));
}

__device__ __forceinline__ float wave_max(float v) {
    v = row16_max(v);
    return fmaxf(fmaxf(read_lane(v, 0), read_lane(v, 16)), fmaxf(read_lane(v, 32), read_lane(v, 48)));
}

// Workgroup barrier for data that travels through LDS only: orders LDS accesses and leaves global
// loads that are still in flight alone (a full __syncthreads() waits for those as well).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
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
