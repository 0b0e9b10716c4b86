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

// The quantised matmul with its neighbours of a decoder layer inside the launch: where the activations come
// from and where the result goes (one activation row).  Tensors that a kind does not use stay empty.
struct MatmulChain {
    enum class In { Row, SwiGLU, AttentionChunks, NormFromTileSums };
    enum class Out { Row, Residual, QkvRope };
    In in = In::Row;
    Out out = Out::Row;
    tensor::Tensor x;                                 // In::Row: bf16 [K]
    tensor::Tensor gate, up;                          // In::SwiGLU: bf16 [K] each, x = bf16(silu(gate)) * up
    tensor::Tensor attention_chunks;                  // In::AttentionChunks: what MultiHeadAttention::forward_chunks left
    int32_t n_q_heads = 0, n_kv_heads = 0, max_positions = 0;
    tensor::Tensor norm_row, norm_tile_sumsq, norm_gain;  // In::NormFromTileSums: x = gain * bf16(row * rsqrt(mean + eps)),
    float norm_eps = 0.0f;                                 // the row's sums of squares given per quarter of 256 columns
    tensor::Tensor y;                                 // Out::Row: bf16 [N]
    tensor::Tensor residual, tile_sumsq;              // Out::Residual: residual <- bf16(residual + bf16(y)) in place,
                                                      // fp32 [ceil(N / 256), 4] sums of squares of the new row
    tensor::Tensor q_gain, k_gain, q_out, k_cache, v_cache, pos;  // Out::QkvRope: as RoPEKernel below
    int32_t rope_n_q_heads = 0, rope_n_kv_heads = 0;
    float rope_theta = 0.0f, qk_eps = 0.0f;
};
using MatmulChainKernel = void (*)(const MatmulChain& chain, const tensor::Tensor& qweight, const tensor::Tensor& scales,
                                   const tensor::Tensor& qzeros, int32_t group_size, void* stream);
MatmulChainKernel get_matmul_chain_kernel(base::DeviceType device_type);

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
// holds the per-chunk results; with an empty `output` the GPU kernel stops there (the chunks are then merged
// by the consumer, MatmulChain::In::AttentionChunks)
using MhaKernel = void (*)(const tensor::Tensor& q, const tensor::Tensor& k_cache, const tensor::Tensor& v_cache,
                           const tensor::Tensor& pos, const tensor::Tensor& workspace, const tensor::Tensor& output,
                           int32_t n_q_heads, int32_t n_kv_heads, void* stream);
MhaKernel get_mha_kernel(base::DeviceType device_type);

}  // namespace kernel

#endif  // KERNEL_INTERFACE_H
