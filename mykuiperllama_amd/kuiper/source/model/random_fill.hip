// Fill kernels for random-init models (see random_fill.h).  Byte movers: one element per thread
// and step of a grid-stride loop, 16-bit and 32-bit stores that a wave issues side by side.
#include "random_fill.h"

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "base/base.h"

namespace model {
namespace {

__device__ __forceinline__ uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__device__ __forceinline__ float unit_interval(uint64_t bits) {  // [0, 1) from the top 24 bits
    return static_cast<float>(bits >> 40) * (1.0f / 16777216.0f);
}

__device__ __forceinline__ uint16_t to_bf16(float f) {  // finite input, round to nearest even
    uint32_t u = __float_as_uint(f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

__global__ __launch_bounds__(256) void words_kernel(uint32_t* __restrict__ p, size_t n, uint64_t seed) {
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
        p[i] = static_cast<uint32_t>(splitmix64(seed + i));
    }
}

__global__ __launch_bounds__(256) void uniform_fp16_kernel(uint16_t* __restrict__ p, size_t n, uint64_t seed, float low,
                                                          float span) {
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
        const __half h = __float2half(low + span * unit_interval(splitmix64(seed + i)));
        p[i] = __half_as_ushort(h);
    }
}

__global__ __launch_bounds__(256) void normal_bf16_kernel(uint16_t* __restrict__ p, size_t n, uint64_t seed, float mean,
                                                         float std) {
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint64_t bits = splitmix64(seed + i);
        const float u1 = 1.0f - unit_interval(bits);                    // (0, 1]
        const float u2 = unit_interval(splitmix64(bits ^ 0xD1B54A32D192ED03ull));
        const float z = sqrtf(-2.0f * logf(u1)) * cosf(6.28318530718f * u2);
        p[i] = to_bf16(mean + std * z);
    }
}

unsigned blocks_for(size_t n) {
    size_t blocks = (n + 255) / 256;
    if (blocks > 16384) blocks = 16384;  // the grid-stride loop takes the rest
    return static_cast<unsigned>(blocks == 0 ? 1 : blocks);
}

void check_launch(const char* what) {
    const hipError_t err = hipGetLastError();
    CHECK(err == hipSuccess) << what << " launch failed: " << hipGetErrorString(err);
}

}  // namespace

void fill_random_words(int32_t* device_ptr, size_t n, uint64_t seed, void* stream) {
    CHECK_NE(device_ptr, nullptr);
    hipLaunchKernelGGL(words_kernel, dim3(blocks_for(n)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<uint32_t*>(device_ptr), n, seed);
    check_launch("random words");
}

void fill_uniform_fp16(uint16_t* device_ptr, size_t n, uint64_t seed, float low, float high, void* stream) {
    CHECK_NE(device_ptr, nullptr);
    hipLaunchKernelGGL(uniform_fp16_kernel, dim3(blocks_for(n)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       device_ptr, n, seed, low, high - low);
    check_launch("uniform fp16");
}

void fill_normal_bf16(uint16_t* device_ptr, size_t n, uint64_t seed, float mean, float std, void* stream) {
    CHECK_NE(device_ptr, nullptr);
    hipLaunchKernelGGL(normal_bf16_kernel, dim3(blocks_for(n)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       device_ptr, n, seed, mean, std);
    check_launch("normal bf16");
}

}  // namespace model
