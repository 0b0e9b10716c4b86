// RmsNormLayer: y = gain * bf16(x * rsqrt(mean(x^2) + eps)) over the last dimension, bf16 tensors
// (the LayerRMSNorm slot, kuiper/include/op/layer.h:12; the reference's rmsnorm.h is an empty
// namespace).  With two inputs the second is a residual delta: input 0 is updated in place,
// x <- bf16(x + delta), and the norm is taken of the updated rows.
//   weight 0   gain bf16 [dim]
//   input 0    x bf16 [rows, dim] or [dim]      input 1 (optional)   delta, same shape
//   output 0   y, same shape
#ifndef KUIPER_INCLUDE_OP_RMSNORM_H
#define KUIPER_INCLUDE_OP_RMSNORM_H

#include "op/typed_layer.h"

namespace op {

class RmsNormLayer : public TypedLayer {
public:
    explicit RmsNormLayer(base::DeviceType device_type, int32_t dim, float eps = 1e-6f);
    base::Status check() const override;
    base::Status forward() override;
    using TypedLayer::forward;

private:
    int32_t dim_ = 0;
    float eps_ = 1e-6f;
};

}  // namespace op

#endif  // KUIPER_INCLUDE_OP_RMSNORM_H
