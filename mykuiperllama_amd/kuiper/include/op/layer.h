// Operator layer interfaces of the kuiper host API: BaseLayer (pure interface), Layer (inputs,
// outputs, stream config), LayerParam (weights plus the quantisation members).  Names, virtual
// signatures, defaults and checks follow kuiper/include/op/layer.h:8-156 and
// kuiper/source/op/layer.cpp of the reference.
#ifndef KUIPER_INCLUDE_OP_LAYER_H
#define KUIPER_INCLUDE_OP_LAYER_H

#include <memory>
#include <string>
#include <vector>

#include "base/cuda_config.h"
#include "tensor/tensor.h"

namespace op {

enum class LayerType : uint8_t {
    LayerUnknown = 0,
    LayerLinear = 1,
    LayerEncode = 2,
    LayerEmbedding = 3,
    LayerRMSNorm = 4,
    LayerMatmul = 5,
    LayerRope = 6,
    LayerMHA = 7,
    LayerSoftmax = 8,
    LayerAdd = 9,
    LayerSwiGLU = 10,
};

class BaseLayer {
public:
    explicit BaseLayer(base::DeviceType device_type, LayerType layer_type, base::DataType data_type,
                       std::string layer_name = "");
    virtual ~BaseLayer() = default;

    virtual base::Status init() = 0;
    virtual base::Status check() const = 0;

    virtual base::Status forward() = 0;
    virtual base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& output1) = 0;
    virtual base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2,
                                 const tensor::Tensor& output1) = 0;
    virtual base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2,
                                 const tensor::Tensor& input3, const tensor::Tensor& output1) = 0;
    virtual base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2,
                                 const tensor::Tensor& input3, const tensor::Tensor& input4,
                                 const tensor::Tensor& output1) = 0;
    virtual base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2,
                                 const tensor::Tensor& input3, const tensor::Tensor& input4,
                                 const tensor::Tensor& input5, const tensor::Tensor& output1) = 0;

    virtual void set_input(int32_t idx, const tensor::Tensor& input) = 0;
    virtual void set_output(int32_t idx, const tensor::Tensor& output) = 0;
    virtual size_t input_size() const = 0;
    virtual size_t output_size() const = 0;
    virtual tensor::Tensor& get_input(int32_t idx) = 0;
    virtual tensor::Tensor& get_output(int32_t idx) = 0;
    virtual const tensor::Tensor& get_input(int32_t idx) const = 0;
    virtual const tensor::Tensor& get_output(int32_t idx) const = 0;

    // Layers without weights answer "not implemented".
    virtual base::Status set_weight(int32_t idx, const tensor::Tensor& weight);
    virtual base::Status set_weight(int32_t idx, const std::vector<int32_t>& dims, const void* weight_ptr,
                                    base::DeviceType device_type = base::DeviceType::DeviceUnknown);

    const std::string& layer_name() const;
    LayerType layer_type() const;
    base::DataType data_type() const;
    base::DeviceType device_type() const;
    void set_layer_name(const std::string& layer_name);
    void set_device_type(base::DeviceType device_type);

protected:
    std::string layer_name_;
    LayerType layer_type_ = LayerType::LayerUnknown;
    base::DataType data_type_ = base::DataType::DataTypeUnknown;
    base::DeviceType device_type_ = base::DeviceType::DeviceUnknown;
};

// A layer without weights.  Its element type is fp32 (reference layer.cpp:41-42); layers that
// compute in another type override set_input / set_output.
class Layer : public BaseLayer {
public:
    explicit Layer(base::DeviceType device_type, LayerType layer_type, std::string layer_name = "");

    base::Status init() override;
    base::Status check() const override;

    base::Status check_tensor(const tensor::Tensor& tensor, base::DeviceType device_type,
                              base::DataType data_type) const;
    // Followed by one int32_t per dimension of `tensor`: the expected extents.
    base::Status check_tensor_with_dim(const tensor::Tensor& tensor, base::DeviceType device_type,
                                       base::DataType data_type, ...) const;

    base::Status forward() override;
    base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& output1) override;
    base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2,
                         const tensor::Tensor& output1) override;
    base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2,
                         const tensor::Tensor& input3, const tensor::Tensor& output1) override;
    base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2,
                         const tensor::Tensor& input3, const tensor::Tensor& input4,
                         const tensor::Tensor& output1) override;
    base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2,
                         const tensor::Tensor& input3, const tensor::Tensor& input4,
                         const tensor::Tensor& input5, const tensor::Tensor& output1) override;

    void set_input(int32_t idx, const tensor::Tensor& input) override;
    void set_output(int32_t idx, const tensor::Tensor& output) override;
    size_t input_size() const override;
    size_t output_size() const override;
    tensor::Tensor& get_input(int32_t idx) override;
    tensor::Tensor& get_output(int32_t idx) override;
    const tensor::Tensor& get_input(int32_t idx) const override;
    const tensor::Tensor& get_output(int32_t idx) const override;

    void reset_input_size(size_t size);
    void reset_output_size(size_t size);

    void set_cuda_config(std::shared_ptr<kernel::CudaConfig> cuda_config);  // a null config is ignored
    std::shared_ptr<kernel::CudaConfig> cuda_config() const;

    virtual void to_cuda();  // moves every non-empty input and output to the GPU

protected:
    std::vector<tensor::Tensor> inputs_;
    std::vector<tensor::Tensor> outputs_;
    std::shared_ptr<kernel::CudaConfig> cuda_config_;
};

// A layer with weights, and the members a group-quantised layer needs.
class LayerParam : public Layer {
public:
    explicit LayerParam(base::DeviceType device_type, LayerType layer_type, bool is_quant_layer = false,
                        std::string layer_name = "");

    size_t weights_size() const;
    void reset_weights_size(size_t size);
    tensor::Tensor& get_weight(int32_t idx);
    const tensor::Tensor& get_weight(int32_t idx) const;

    // fp32 weights only at this level (reference layer.cpp:248); typed layers override.
    base::Status set_weight(int32_t idx, const tensor::Tensor& weight) override;
    // Borrows weight_ptr (no copy) as an fp32 tensor of `dims`; a quantised layer stores nothing
    // here (reference layer.cpp:256-276) and leaves the attach to its own override.
    base::Status set_weight(int32_t idx, const std::vector<int32_t>& dims, const void* weight_ptr,
                            base::DeviceType device_type = base::DeviceType::DeviceUnknown) override;

    void set_scales(const tensor::Tensor& scales);  // same element type and device as the layer
    void set_group_size(int32_t group_size);
    int32_t get_scale_num() const;

    void to_cuda() override;  // also moves weights and scales

protected:
    int32_t group_size_ = 0;
    bool is_quant_layer_ = false;
    tensor::Tensor scales_;
    std::vector<tensor::Tensor> weights_;
};

}  // namespace op

#endif  // KUIPER_INCLUDE_OP_LAYER_H
