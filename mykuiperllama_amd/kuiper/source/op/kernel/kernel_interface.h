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

// Decode-step operators (the layer slots LayerRMSNorm, LayerSwiGLU, LayerEmbedding, LayerRope,
// LayerMHA of kuiper/include/op/layer.h:8-20); bf16 tensors, head_dim 128.
// y = gain * bf16(r * rsqrt(mean(r^2) + eps)) over the last dimension; with a non-empty `delta` the
// input is first updated in place, r = input <- bf16(input + delta) (the residual add)
using RmsNormKernel = void (*)(const tensor::Tensor& input, const tensor::Tensor& delta,
                               const tensor::Tensor& weight, const tensor::Tensor& output, float eps,
                               void* stream);
RmsNormKernel get_rmsnorm_kernel(base::DeviceType device_type);

// out = bf16(silu(gate)) * up
using SwiGLUKernel = void (*)(const tensor::Tensor& gate, const tensor::Tensor& up, const tensor::Tensor& output,
                              void* stream);
SwiGLUKernel get_swiglu_kernel(base::DeviceType device_type);

// out = table[token[0], :]; token int32 [1] on the layer's device, clamped to the vocabulary
using EmbeddingKernel = void (*)(const tensor::Tensor& token, const tensor::Tensor& table,
                                 const tensor::Tensor& output, void* stream);
EmbeddingKernel get_embedding_kernel(base::DeviceType device_type);

// qkv = [q heads | k heads | v heads] x 128: per-head RMSNorm of q and k, rotation at pos[0] (int32 [1] on
// the device), q to q_out, k and v into row pos[0] of the caches [max_positions, n_kv_heads, 128]
using RoPEKernel = void (*)(const tensor::Tensor& qkv, const tensor::Tensor& q_gain, const tensor::Tensor& k_gain,
                            const tensor::Tensor& pos, const tensor::Tensor& q_out, const tensor::Tensor& k_cache,
                            const tensor::Tensor& v_cache, int32_t n_q_heads, int32_t n_kv_heads, float theta,
                            float eps, void* stream);
RoPEKernel get_rope_kernel(base::DeviceType device_type);

// grouped-query attention of one query position against cache rows 0 .. pos[0]; `workspace` (GPU only)
// holds the per-chunk results
using MhaKernel = void (*)(const tensor::Tensor& q, const tensor::Tensor& k_cache, const tensor::Tensor& v_cache,
                           const tensor::Tensor& pos, const tensor::Tensor& workspace, const tensor::Tensor& output,
                           int32_t n_q_heads, int32_t n_kv_heads, void* stream);
MhaKernel get_mha_kernel(base::DeviceType device_type);

}  // namespace kernel

#endif  // KERNEL_INTERFACE_H
