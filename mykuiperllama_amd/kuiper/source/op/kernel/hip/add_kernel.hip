// GPU add kernel (reference: kuiper/source/op/kernel/cuda/add_kernel.cu:4-52, one element per
// thread).  Here each thread moves 16 bytes and a grid-stride loop covers the tail, so a wave
// reads and writes whole 1 KiB lines; the arithmetic is the same single fp32 addition per
// element.
#include <hip/hip_runtime.h>

#include "add_kernel.h"

namespace kernel {
namespace {

__global__ __launch_bounds__(256) void add_fp32_kernel(size_t n, const float* __restrict__ a,
                                                       const float* __restrict__ b, float* __restrict__ out) {
    const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    const size_t n4 = n / 4;
    const float4* a4 = reinterpret_cast<const float4*>(a);
    const float4* b4 = reinterpret_cast<const float4*>(b);
    float4* o4 = reinterpret_cast<float4*>(out);
    for (size_t i = tid; i < n4; i += stride) {
        const float4 x = a4[i];
        const float4 y = b4[i];
        o4[i] = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
    }
    for (size_t i = 4 * n4 + tid; i < n; i += stride) {
        out[i] = a[i] + b[i];
    }
}

}  // namespace

void add_kernel_cu(const tensor::Tensor& input1, const tensor::Tensor& input2,
                   const tensor::Tensor& output, void* stream) {
    CHECK(input1.device_type() == base::DeviceType::DeviceCUDA);
    CHECK(input2.device_type() == base::DeviceType::DeviceCUDA);
    CHECK(output.device_type() == base::DeviceType::DeviceCUDA);
    CHECK_EQ(input1.is_empty(), false);
    CHECK_EQ(input2.is_empty(), false);
    CHECK_EQ(output.is_empty(), false);
    const size_t n = output.size();
    CHECK_EQ(input1.size(), n);
    CHECK_EQ(input2.size(), n);

    const size_t work = (n + 3) / 4;
    size_t blocks = (work + 255) / 256;
    if (blocks > 4096) blocks = 4096;  // the grid-stride loop takes the rest
    hipLaunchKernelGGL(add_fp32_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), n, input1.ptr<float>(), input2.ptr<float>(),
                       const_cast<float*>(output.ptr<float>()));
    hipError_t err = hipGetLastError();
    CHECK(err == hipSuccess) << "ADD kernel launch failed: " << hipGetErrorString(err);
}

}  // namespace kernel
