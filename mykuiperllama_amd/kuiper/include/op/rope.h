// RoPELayer: what follows the fused q|k|v projection of a Qwen3-style layer (the LayerRope slot,
// kuiper/include/op/layer.h:14; the reference's rope.h is an empty namespace): RMSNorm over each
// query and key head with a 128-element gain, rotary embedding at the current position (rotate-half
// convention, frequencies theta^(-i/64)), queries to the output, keys and values into row `pos` of
// the caches.  head_dim is 128.
//   weight 0   q_gain bf16 [128]       weight 1   k_gain bf16 [128]
//   input 0    qkv bf16 [(n_q + 2 n_kv) * 128]   (query heads, then key heads, then value heads)
//   input 1    pos int32 [1] on the layer's device
//   input 2    k_cache bf16 [max_positions, n_kv, 128]     input 3   v_cache, same shape   (row pos is written)
//   output 0   q bf16 [n_q * 128]
#ifndef KUIPER_INCLUDE_OP_ROPE_H
#define KUIPER_INCLUDE_OP_ROPE_H

#include "op/typed_layer.h"

namespace op {

class RoPELayer : public TypedLayer {
public:
    explicit RoPELayer(base::DeviceType device_type, int32_t n_q_heads, int32_t n_kv_heads, float theta = 1e6f,
                       float eps = 1e-6f);
    base::Status check() const override;
    base::Status forward() override;
    using TypedLayer::forward;

private:
    int32_t n_q_ = 0;
    int32_t n_kv_ = 0;
    float theta_ = 1e6f;
    float eps_ = 1e-6f;
};

}  // namespace op

#endif  // KUIPER_INCLUDE_OP_ROPE_H
