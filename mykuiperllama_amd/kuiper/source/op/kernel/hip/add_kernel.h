#ifndef KUIPER_KERNEL_HIP_ADD_KERNEL_H
#define KUIPER_KERNEL_HIP_ADD_KERNEL_H

#include "tensor/tensor.h"

namespace kernel {
// out[i] = in1[i] + in2[i] on the GPU, fp32.  Enqueued on `stream` (a hipStream_t; nullptr = the
// default stream); no synchronisation.
void add_kernel_cu(const tensor::Tensor& input1, const tensor::Tensor& input2,
                   const tensor::Tensor& output, void* stream);
}  // namespace kernel

#endif  // KUIPER_KERNEL_HIP_ADD_KERNEL_H
