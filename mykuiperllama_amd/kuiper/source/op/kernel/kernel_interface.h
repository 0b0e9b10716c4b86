// Device -> kernel selection, one function-pointer type per operator
// (reference: kuiper/source/op/kernel/kernel_interface.h:10-11 for the add operator; the two
// matmul entries are the ones its empty matmul.h calls for).  The output is passed as a const
// reference and written through, as in the reference's wrappers.
#ifndef KERNEL_INTERFACE_H
#define KERNEL_INTERFACE_H

#include "tensor/tensor.h"

namespace kernel {

using AddKernel = void (*)(const tensor::Tensor& input1, const tensor::Tensor& input2,
                           const tensor::Tensor& output, void* stream);
AddKernel get_add_kernel(base::DeviceType device_type);

// y[M,N] = x[M,K] * W[N,K]^T, all bf16, fp32 accumulation
using MatmulKernel = void (*)(const tensor::Tensor& input, const tensor::Tensor& weight,
                              const tensor::Tensor& output, void* stream);
MatmulKernel get_matmul_kernel(base::DeviceType device_type);

// y[M,N] = x[M,K] * dequant(qweight, scales, qzeros)[K,N]; x, y bf16; qweight int32 [K,N/8];
// scales fp16 [K/G,N]; qzeros int32 [K/G,N/8]
using MatmulKernelAwq = void (*)(const tensor::Tensor& input, const tensor::Tensor& qweight,
                                 const tensor::Tensor& scales, const tensor::Tensor& qzeros,
                                 const tensor::Tensor& output, int32_t group_size, void* stream);
MatmulKernelAwq get_matmul_kernel_awq(base::DeviceType device_type);

}  // namespace kernel

#endif  // KERNEL_INTERFACE_H
