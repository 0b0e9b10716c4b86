// VecAddLayer: out = in1 + in2 over fp32 tensors (reference: kuiper/include/op/add.h:7-14).
#ifndef KUIPER_INCLUDE_OP_ADD_H
#define KUIPER_INCLUDE_OP_ADD_H

#include "op/layer.h"

namespace op {

class VecAddLayer : public Layer {
public:
    explicit VecAddLayer(base::DeviceType device_type);
    base::Status check() const override;
    base::Status forward() override;
    using Layer::forward;  // keep the forward(inputs..., output) overloads visible on this type
};

}  // namespace op

#endif  // KUIPER_INCLUDE_OP_ADD_H
