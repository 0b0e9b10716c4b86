// Base of the layers whose tensors are not fp32: Layer / LayerParam insist on the layer's one element
// type (kuiper/source/op/layer.cpp:138-156, :245-253 of the reference, fp32 there); a decode-step
// operator mixes bf16 activations with int32 scalars (token, position), so this base accepts any
// element type on a slot, still requires the layer's device, and leaves the typing to check().
#ifndef KUIPER_INCLUDE_OP_TYPED_LAYER_H
#define KUIPER_INCLUDE_OP_TYPED_LAYER_H

#include "op/layer.h"

namespace op {

class TypedLayer : public LayerParam {
public:
    explicit TypedLayer(base::DeviceType device_type, LayerType layer_type, std::string layer_name);

    void set_input(int32_t idx, const tensor::Tensor& input) override;
    void set_output(int32_t idx, const tensor::Tensor& output) override;
    base::Status set_weight(int32_t idx, const tensor::Tensor& weight) override;  // bf16, layer's device
    using LayerParam::set_weight;
    using Layer::forward;  // keep the forward(inputs..., output) overloads visible

protected:
    void* stream() const;  // the layer's stream, or null
    // bf16 (or int32) tensor of exactly `elements` elements on the layer's device
    base::Status expect(const tensor::Tensor& t, base::DataType type, size_t elements, const char* what) const;
};

}  // namespace op

#endif  // KUIPER_INCLUDE_OP_TYPED_LAYER_H
