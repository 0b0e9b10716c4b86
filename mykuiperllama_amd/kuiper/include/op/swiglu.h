// SwiGLULayer: out = bf16(silu(gate)) * up over bf16 tensors of `dim` elements (the LayerSwiGLU slot,
// kuiper/include/op/layer.h:18; the reference's swiglu.h is an empty namespace).
//   input 0 gate, input 1 up, output 0: bf16 [dim]
#ifndef KUIPER_INCLUDE_OP_SWIGLU_H
#define KUIPER_INCLUDE_OP_SWIGLU_H

#include "op/typed_layer.h"

namespace op {

class SwiGLULayer : public TypedLayer {
public:
    explicit SwiGLULayer(base::DeviceType device_type, int32_t dim);
    base::Status check() const override;
    base::Status forward() override;
    using TypedLayer::forward;

private:
    int32_t dim_ = 0;
};

}  // namespace op

#endif  // KUIPER_INCLUDE_OP_SWIGLU_H
