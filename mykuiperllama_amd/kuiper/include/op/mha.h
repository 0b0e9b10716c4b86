// MultiHeadAttention: grouped-query attention of one query position against cache rows 0 .. pos
// (the LayerMHA slot, kuiper/include/op/layer.h:15; the reference's mha.h is an empty namespace).
// out[h, :] = softmax(q[h, :] . K[:, h / G, :] / sqrt(128)) V[:, h / G, :], G = n_q / n_kv between 1 and 16.
//   input 0    q bf16 [n_q * 128]
//   input 1    pos int32 [1] on the layer's device
//   input 2    k_cache bf16 [max_positions, n_kv, 128]     input 3   v_cache, same shape
//   output 0   bf16 [n_q * 128]
// A GPU layer owns the workspace of the split over the context (allocated on first use for the
// cache's max_positions, at most 32768).
#ifndef KUIPER_INCLUDE_OP_MHA_H
#define KUIPER_INCLUDE_OP_MHA_H

#include "op/typed_layer.h"

namespace op {

class MultiHeadAttention : public TypedLayer {
public:
    explicit MultiHeadAttention(base::DeviceType device_type, int32_t n_q_heads, int32_t n_kv_heads);
    base::Status check() const override;
    base::Status forward() override;
    using TypedLayer::forward;
    // GPU only: the first stage alone.  Inputs 0..3 as for forward(); the per-chunk results stay in chunks(), for
    // a MatmulLayer whose fused launch merges them on its way in (kernel::MatmulChain::In::AttentionChunks).
    base::Status forward_chunks(const tensor::Tensor& q, const tensor::Tensor& pos, const tensor::Tensor& k_cache,
                                const tensor::Tensor& v_cache);
    const tensor::Tensor& chunks() const { return workspace_; }
    // Allocates the GPU workspace for caches of max_positions rows now, so that forward() allocates
    // nothing later (a stream under graph capture must not).  No effect on a host layer.
    base::Status reserve(int32_t max_positions);

private:
    int32_t n_q_ = 0;
    int32_t n_kv_ = 0;
    base::Status grow_workspace(size_t need);

    tensor::Tensor workspace_;  // GPU only
};

}  // namespace op

#endif  // KUIPER_INCLUDE_OP_MHA_H
