#ifndef KUIPER_KERNEL_CPU_ADD_KERNEL_H
#define KUIPER_KERNEL_CPU_ADD_KERNEL_H

#include "tensor/tensor.h"

namespace kernel {
// out[i] = in1[i] + in2[i], fp32, single thread; `stream` is ignored.
void add_kernel_cpu(const tensor::Tensor& input1, const tensor::Tensor& input2,
                    const tensor::Tensor& output, void* stream);
}  // namespace kernel

#endif  // KUIPER_KERNEL_CPU_ADD_KERNEL_H
