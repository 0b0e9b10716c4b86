// MatmulLayer: y = x * W^T for decode-sized batches, the operator the reference reserves the
// LayerMatmul slot for (kuiper/include/op/layer.h:14) and declares no further
// (kuiper/include/op/matmul.h:7-9 is an empty namespace).
//
//   dim0 = output features N, dim1 = input features K   (weights read as [dim0, dim1])
//   input  x  bf16 [M, K] or [K]        output y  bf16 [M, N] or [N],  M <= 16
//
// Unquantised layer (is_quant_layer == false):
//   weight 0   bf16 [N, K]
// INT4 AWQ layer (is_quant_layer == true), group size G along K:
//   weight 0   qweight int32 [K, N/8]     eight 4-bit codes per word, column order 0,2,4,6,1,3,5,7
//   weight 1   qzeros  int32 [K/G, N/8]   same packing
//   scales     fp16 [K/G, N]              set_awq_scales()
//   w[k,n] = (q[k,n] - z[k/G,n]) * s[k/G,n]
//
// forward() follows the pattern of VecAddLayer::forward (kuiper/source/op/add.cpp:36-49): check(),
// then kernel::get_matmul_kernel[_awq](device_type_)(..., stream).  No synchronisation inside.
//
// A GPU AWQ layer can take its neighbours in a decoder layer into its launch (set_fusion): the
// activations produced on the way in (SwiGLU of two rows, RMSNorm from the row's tile sums of squares, the
// merge of the attention chunks) and the result consumed on the way out (residual add with the new row's
// tile sums, or per-head norm + rotation + KV-cache append of a q|k|v row).  forward() then goes through
// kernel::get_matmul_chain_kernel(device_type_); input 0 / output 0 are used only by the ends that stay
// plain rows.  One activation row.  This is the quantised-layer hook the reference reserves in
// kuiper/include/op/layer.h:122-156 (scales, group size on LayerParam), extended to the launches
// themselves.
#ifndef KUIPER_INCLUDE_OP_MATMUL_H
#define KUIPER_INCLUDE_OP_MATMUL_H

#include <memory>

#include "base/cuda_config.h"
#include "op/layer.h"

namespace kernel {
struct MatmulChain;
}

namespace op {

class MatmulLayer : public LayerParam {
public:
    explicit MatmulLayer(base::DeviceType device_type, int32_t dim0, int32_t dim1,
                         bool is_quant_layer = false, int32_t group_size = 128);

    base::Status check() const override;
    base::Status forward() override;
    using Layer::forward;  // keep the forward(inputs..., output) overloads visible on this type

    // Activations are bf16 here, not the fp32 that Layer assumes.
    void set_input(int32_t idx, const tensor::Tensor& input) override;
    void set_output(int32_t idx, const tensor::Tensor& output) override;

    // Typed by slot: bf16 for slot 0 of an unquantised layer, int32 for both slots of an AWQ layer.
    base::Status set_weight(int32_t idx, const tensor::Tensor& weight) override;
    // Borrows weight_ptr with the slot's element type (no copy).
    base::Status set_weight(int32_t idx, const std::vector<int32_t>& dims, const void* weight_ptr,
                            base::DeviceType device_type = base::DeviceType::DeviceUnknown) override;

    // fp16 scales of an AWQ layer.  LayerParam::set_scales is not virtual and insists on the
    // layer's own element type, so the fp16 tensor comes in through this method.
    void set_awq_scales(const tensor::Tensor& scales);
    const tensor::Tensor& awq_scales() const;

    // The fused form of this layer's launch: what kernel::MatmulChain describes (its x / y are ignored when the
    // corresponding end is a plain row: input 0 / output 0 of the layer are used).  GPU AWQ layers only.
    base::Status set_fusion(const kernel::MatmulChain& chain);
    void clear_fusion();
    bool fused() const;

    int32_t dim0() const;
    int32_t dim1() const;
    int32_t group_size() const;
    bool is_quant_layer() const;

private:
    base::Status forward_fused();

    int32_t dim0_ = 0;  // N
    int32_t dim1_ = 0;  // K
    std::shared_ptr<kernel::MatmulChain> fusion_;
};

}  // namespace op

#endif  // KUIPER_INCLUDE_OP_MATMUL_H
