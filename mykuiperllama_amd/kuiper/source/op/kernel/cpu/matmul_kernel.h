#ifndef KUIPER_KERNEL_CPU_MATMUL_KERNEL_H
#define KUIPER_KERNEL_CPU_MATMUL_KERNEL_H

#include "tensor/tensor.h"

namespace kernel {

// Host kernels of the matmul operator, selected only when a layer is constructed for DeviceCPU.
// Single thread, `stream` ignored, in the manner of the reference's host kernels
// (kuiper/source/op/kernel/cpu/add_kernel.cpp:5-26).  The GPU path never routes through them.
void matmul_kernel_cpu(const tensor::Tensor& input, const tensor::Tensor& weight,
                       const tensor::Tensor& output, void* stream);
void matmul_kernel_awq_cpu(const tensor::Tensor& input, const tensor::Tensor& qweight,
                           const tensor::Tensor& scales, const tensor::Tensor& qzeros,
                           const tensor::Tensor& output, int32_t group_size, void* stream);

}  // namespace kernel

#endif  // KUIPER_KERNEL_CPU_MATMUL_KERNEL_H
