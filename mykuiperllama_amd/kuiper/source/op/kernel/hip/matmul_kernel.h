#ifndef KUIPER_KERNEL_HIP_MATMUL_KERNEL_H
#define KUIPER_KERNEL_HIP_MATMUL_KERNEL_H

#include "tensor/tensor.h"

namespace kernel {

// GPU kernels of the matmul operator: thin wrappers that check the tensors the way the
// reference's GPU wrapper does (kuiper/source/op/kernel/cuda/add_kernel.cu:14-52: device, non-empty,
// sizes; then launch; then a fatal check of the launch status; no synchronisation) and call the
// C ABI of the HIP library (include/kx_hip.h).  The split-K workspace is kept per stream and
// grows on demand; it is the only allocation these wrappers ever make.
void matmul_kernel_cu(const tensor::Tensor& input, const tensor::Tensor& weight,
                      const tensor::Tensor& output, void* stream);
void matmul_kernel_awq_cu(const tensor::Tensor& input, const tensor::Tensor& qweight,
                          const tensor::Tensor& scales, const tensor::Tensor& qzeros,
                          const tensor::Tensor& output, int32_t group_size, void* stream);

struct MatmulChain;
// One fused launch of a decoder layer (kx_gemv_awq_chain_bf16), one activation row.
void matmul_chain_kernel_cu(const MatmulChain& chain, const tensor::Tensor& qweight, const tensor::Tensor& scales,
                            const tensor::Tensor& qzeros, int32_t group_size, void* stream);

// Releases every cached workspace (for orderly shutdown in tests).
void matmul_release_workspaces();
// Releases the workspace of one stream; whoever destroys a stream calls this first, so that a later
// stream that happens to get the same handle starts without an entry.
void matmul_release_workspace(void* stream);

// Makes the workspace of `stream` large enough for a GEMV of this shape now, so that later launches
// on that stream allocate nothing (a stream under graph capture must not).
void matmul_reserve_workspace(void* stream, int32_t M, int32_t K, int32_t N);

}  // namespace kernel

#endif  // KUIPER_KERNEL_HIP_MATMUL_KERNEL_H
