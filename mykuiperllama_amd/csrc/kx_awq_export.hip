// Export kernels for the integer side of the AWQ path: unpacked codes and dequantised bf16
// weights, written the plain way (one thread per packed word) so that they can serve as the
// bit-exact witness for the nibble order and for w = (q - z) * s.
#include "kx_common.h"

namespace kx {
namespace {

__global__ __launch_bounds__(256) void awq_unpack_kernel(const uint32_t* __restrict__ words,
                                                         uint8_t* __restrict__ codes, size_t nwords) {
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= nwords) return;
    uint32_t w = words[i];
    uint8_t out[8];
#pragma unroll
    for (int nib = 0; nib < 8; nib++) {
        out[order_of(nib)] = static_cast<uint8_t>((w >> (4 * nib)) & 0xfu);
    }
    uint2 packed;
    packed.x = out[0] | (out[1] << 8) | (out[2] << 16) | (static_cast<uint32_t>(out[3]) << 24);
    packed.y = out[4] | (out[5] << 8) | (out[6] << 16) | (static_cast<uint32_t>(out[7]) << 24);
    reinterpret_cast<uint2*>(codes)[i] = packed;  // word i covers codes[8i .. 8i+7]
}

__global__ __launch_bounds__(256) void awq_dequant_kernel(const uint32_t* __restrict__ qweight,
                                                          const uint16_t* __restrict__ scales,
                                                          const uint32_t* __restrict__ qzeros,
                                                          uint16_t* __restrict__ w, int K, int N,
                                                          int group) {
    const int nw = N >> 3;
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= static_cast<size_t>(K) * nw) return;
    const int k = static_cast<int>(i / nw);
    const int j = static_cast<int>(i % nw);
    const int g = k / group;
    const uint32_t qw = qweight[i];
    const uint32_t zw = qzeros[static_cast<size_t>(g) * nw + j];
    const uint16_t* sp = scales + static_cast<size_t>(g) * N + 8 * j;
    uint16_t out[8];
#pragma unroll
    for (int nib = 0; nib < 8; nib++) {
        const int c = order_of(nib);
        const int d = static_cast<int>((qw >> (4 * nib)) & 0xfu) - static_cast<int>((zw >> (4 * nib)) & 0xfu);
        // |d| <= 15 times an 11-bit significand: the fp32 product is exact, the store rounds once.
        out[c] = f32_to_bf16(static_cast<float>(d) * f16_bits_to_f32(sp[c]));
    }
    uint4 packed;
    packed.x = out[0] | (static_cast<uint32_t>(out[1]) << 16);
    packed.y = out[2] | (static_cast<uint32_t>(out[3]) << 16);
    packed.z = out[4] | (static_cast<uint32_t>(out[5]) << 16);
    packed.w = out[6] | (static_cast<uint32_t>(out[7]) << 16);
    reinterpret_cast<uint4*>(w)[i] = packed;  // word (k, j) covers w[k, 8j .. 8j+7]
}

}  // namespace
}  // namespace kx

extern "C" int kx_awq_unpack_u8(const int32_t* words, uint8_t* codes, int64_t rows, int64_t cols,
                                void* stream) {
    if (rows < 0 || cols < 0 || (cols % 8) != 0) return KX_ERR_BAD_SHAPE;
    if (rows == 0 || cols == 0) return KX_OK;
    if (!words || !codes) return KX_ERR_NULL_POINTER;
    if (reinterpret_cast<uintptr_t>(words) % 4 || reinterpret_cast<uintptr_t>(codes) % 8) return KX_ERR_ALIGNMENT;
    size_t nwords = static_cast<size_t>(rows) * static_cast<size_t>(cols / 8);
    size_t blocks = (nwords + 255) / 256;
    if (blocks > 0x7fffffffu) return KX_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(kx::awq_unpack_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       kx::as_stream(stream), reinterpret_cast<const uint32_t*>(words), codes, nwords);
    return kx::launch_status();
}

extern "C" int kx_awq_dequant_bf16(const int32_t* qweight, const uint16_t* scales,
                                   const int32_t* qzeros, uint16_t* w, int32_t K, int32_t N,
                                   int32_t group_size, void* stream) {
    if (!qweight || !scales || !qzeros || !w) return KX_ERR_NULL_POINTER;
    if (K < 1 || N < 8 || (N % 8) != 0 || group_size < 1 || (K % group_size) != 0) return KX_ERR_BAD_SHAPE;
    if (reinterpret_cast<uintptr_t>(w) % 16 || reinterpret_cast<uintptr_t>(qweight) % 4 ||
        reinterpret_cast<uintptr_t>(qzeros) % 4 || reinterpret_cast<uintptr_t>(scales) % 2) {
        return KX_ERR_ALIGNMENT;
    }
    size_t nwords = static_cast<size_t>(K) * static_cast<size_t>(N / 8);
    size_t blocks = (nwords + 255) / 256;
    if (blocks > 0x7fffffffu) return KX_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(kx::awq_dequant_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       kx::as_stream(stream), reinterpret_cast<const uint32_t*>(qweight), scales,
                       reinterpret_cast<const uint32_t*>(qzeros), w, K, N, group_size);
    return kx::launch_status();
}
