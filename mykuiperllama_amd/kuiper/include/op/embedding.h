// EmbeddingLayer: out = table[token, :] (the LayerEmbedding slot, kuiper/include/op/layer.h:11; the
// reference's embedding.h is an empty namespace).  The token id is an int32 tensor on the layer's
// device, so that a captured GPU graph sees new tokens; ids outside the vocabulary are clamped.
//   weight 0   table bf16 [vocab, dim]
//   input 0    token int32 [1]
//   output 0   row bf16 [dim]
#ifndef KUIPER_INCLUDE_OP_EMBEDDING_H
#define KUIPER_INCLUDE_OP_EMBEDDING_H

#include "op/typed_layer.h"

namespace op {

class EmbeddingLayer : public TypedLayer {
public:
    explicit EmbeddingLayer(base::DeviceType device_type, int32_t vocab, int32_t dim);
    base::Status check() const override;
    base::Status forward() override;
    using TypedLayer::forward;

private:
    int32_t vocab_ = 0;
    int32_t dim_ = 0;
};

}  // namespace op

#endif  // KUIPER_INCLUDE_OP_EMBEDDING_H
