#ifndef KUIPER_KERNEL_HIP_DECODE_KERNELS_H
#define KUIPER_KERNEL_HIP_DECODE_KERNELS_H

#include "tensor/tensor.h"

namespace kernel {

// GPU side of the decode-step operators: checks in the manner of the reference's add wrapper
// (kuiper/source/op/kernel/cuda/add_kernel.cu:14-52), then the C ABI of the HIP library on the
// given stream.  No synchronisation.  Argument meaning as in kernel_interface.h.
void rmsnorm_kernel_cu(const tensor::Tensor& input, const tensor::Tensor& delta, const tensor::Tensor& weight,
                       const tensor::Tensor& output, float eps, void* stream);
void swiglu_kernel_cu(const tensor::Tensor& gate, const tensor::Tensor& up, const tensor::Tensor& output,
                      void* stream);
void embedding_kernel_cu(const tensor::Tensor& token, const tensor::Tensor& table, const tensor::Tensor& output,
                         void* stream);
void rope_kernel_cu(const tensor::Tensor& qkv, const tensor::Tensor& q_gain, const tensor::Tensor& k_gain,
                    const tensor::Tensor& pos, const tensor::Tensor& q_out, const tensor::Tensor& k_cache,
                    const tensor::Tensor& v_cache, int32_t n_q_heads, int32_t n_kv_heads, float theta, float eps,
                    void* stream);
void mha_kernel_cu(const tensor::Tensor& q, const tensor::Tensor& k_cache, const tensor::Tensor& v_cache,
                   const tensor::Tensor& pos, const tensor::Tensor& workspace, const tensor::Tensor& output,
                   int32_t n_q_heads, int32_t n_kv_heads, void* stream);

}  // namespace kernel

#endif  // KUIPER_KERNEL_HIP_DECODE_KERNELS_H
