// MatmulLayer: shape checks and dispatch (the reference has no counterpart; the structure follows
// its one concrete layer, kuiper/source/op/add.cpp:5-49).
#include "op/matmul.h"

#include <functional>
#include <numeric>

#include "kernel/kernel_interface.h"

namespace op {
namespace {

constexpr int32_t kMaxBatch = 16;

// [M, K] or [K] -> M; anything else -> -1
int32_t batch_of(const tensor::Tensor& t, int32_t inner) {
    if (t.dims_size() == 1 && t.get_dim(0) == inner) return 1;
    if (t.dims_size() == 2 && t.get_dim(1) == inner) return t.get_dim(0);
    return -1;
}

}  // namespace

MatmulLayer::MatmulLayer(base::DeviceType device_type, int32_t dim0, int32_t dim1, bool is_quant_layer,
                         int32_t group_size)
    : LayerParam(device_type, LayerType::LayerMatmul, is_quant_layer, "Matmul"), dim0_(dim0), dim1_(dim1) {
    data_type_ = base::DataType::DataTypeBf16;  // activations and outputs
    reset_input_size(1);
    reset_output_size(1);
    reset_weights_size(is_quant_layer ? 2 : 1);
    group_size_ = is_quant_layer ? group_size : 0;
}

int32_t MatmulLayer::dim0() const { return dim0_; }
int32_t MatmulLayer::dim1() const { return dim1_; }
int32_t MatmulLayer::group_size() const { return group_size_; }
bool MatmulLayer::is_quant_layer() const { return is_quant_layer_; }
const tensor::Tensor& MatmulLayer::awq_scales() const { return scales_; }

void MatmulLayer::set_input(int32_t idx, const tensor::Tensor& input) {
    CHECK_GE(idx, 0);
    CHECK_LT(static_cast<size_t>(idx), inputs_.size());
    CHECK(input.data_type() == base::DataType::DataTypeBf16);
    if (!input.is_empty()) {
        CHECK(input.device_type() == device_type_);
    }
    inputs_[idx] = input;
}

void MatmulLayer::set_output(int32_t idx, const tensor::Tensor& output) {
    CHECK_GE(idx, 0);
    CHECK_LT(static_cast<size_t>(idx), outputs_.size());
    CHECK(output.data_type() == base::DataType::DataTypeBf16);
    if (!output.is_empty()) {
        CHECK(output.device_type() == device_type_);
    }
    outputs_[idx] = output;
}

base::Status MatmulLayer::set_weight(int32_t idx, const tensor::Tensor& weight) {
    CHECK_GE(idx, 0);
    CHECK_LT(static_cast<size_t>(idx), weights_.size());
    const base::DataType expected = is_quant_layer_ ? base::DataType::DataTypeInt32 : base::DataType::DataTypeBf16;
    CHECK(weight.data_type() == expected);
    if (!weight.is_empty()) {
        CHECK(weight.device_type() == device_type_);
    }
    weights_[idx] = weight;
    return base::error::success();
}

base::Status MatmulLayer::set_weight(int32_t idx, const std::vector<int32_t>& dims, const void* weight_ptr,
                                     base::DeviceType device_type) {
    CHECK_GE(idx, 0);
    CHECK_LT(static_cast<size_t>(idx), weights_.size());
    CHECK_NE(weight_ptr, nullptr);
    const base::DataType type = is_quant_layer_ ? base::DataType::DataTypeInt32 : base::DataType::DataTypeBf16;
    const size_t bytes =
        std::accumulate(dims.begin(), dims.end(), base::data_type_size(type), std::multiplies<size_t>());
    auto borrowed = std::make_shared<base::Buffer>(bytes, nullptr, const_cast<void*>(weight_ptr), true);
    if (device_type != base::DeviceType::DeviceUnknown) {
        borrowed->set_device_type(device_type);
    }
    tensor::Tensor weight;
    weight.reset(type, dims);
    CHECK(weight.assgin(borrowed));
    weights_[idx] = weight;
    return base::error::success();
}

void MatmulLayer::set_awq_scales(const tensor::Tensor& scales) {
    CHECK(is_quant_layer_);
    CHECK(!scales.is_empty());
    CHECK(scales.data_type() == base::DataType::DataTypeFp16);
    CHECK(scales.device_type() == device_type_);
    scales_ = scales;
}

base::Status MatmulLayer::check() const {
    const int32_t N = dim0_;
    const int32_t K = dim1_;
    const tensor::Tensor& x = get_input(0);
    const tensor::Tensor& y = get_output(0);

    base::Status status = check_tensor(x, device_type_, base::DataType::DataTypeBf16);
    if (!status) {
        LOG(ERROR) << "The input tensor error in the matmul layer.";
        return status;
    }
    const int32_t M = batch_of(x, K);
    if (M < 1 || M > kMaxBatch) {
        LOG(ERROR) << "The input tensor error in the matmul layer.";
        return base::error::invalid_argument("The input must be [K] or [M, K] with 1 <= M <= 16.");
    }
    status = check_tensor(y, device_type_, base::DataType::DataTypeBf16);
    if (status && batch_of(y, N) != M) {
        status = base::error::invalid_argument("The output must be [N] or [M, N] with the input's M.");
    }
    if (!status) {
        LOG(ERROR) << "The output tensor error in the matmul layer.";
        return status;
    }

    if (!is_quant_layer_) {
        status = check_tensor_with_dim(get_weight(0), device_type_, base::DataType::DataTypeBf16, N, K);
        if (!status) {
            LOG(ERROR) << "The weight tensor error in the matmul layer.";
        }
        return status;
    }

    const int32_t G = group_size_;
    if (G < 32 || G % 32 != 0 || K % G != 0 || N % 8 != 0) {
        return base::error::invalid_argument(
            "AWQ needs a group size that is a multiple of 32 and divides K, and N a multiple of 8.");
    }
    status = check_tensor_with_dim(get_weight(0), device_type_, base::DataType::DataTypeInt32, K, N / 8);
    if (!status) {
        LOG(ERROR) << "The qweight tensor error in the matmul layer.";
        return status;
    }
    status = check_tensor_with_dim(get_weight(1), device_type_, base::DataType::DataTypeInt32, K / G, N / 8);
    if (!status) {
        LOG(ERROR) << "The qzeros tensor error in the matmul layer.";
        return status;
    }
    status = check_tensor_with_dim(scales_, device_type_, base::DataType::DataTypeFp16, K / G, N);
    if (!status) {
        LOG(ERROR) << "The scales tensor error in the matmul layer.";
    }
    return status;
}

base::Status MatmulLayer::set_fusion(const kernel::MatmulChain& chain) {
    if (!is_quant_layer_ || device_type_ != base::DeviceType::DeviceCUDA) {
        return base::error::invalid_argument("Only a GPU AWQ matmul layer has fused launches.");
    }
    fusion_ = std::make_shared<kernel::MatmulChain>(chain);
    return base::error::success();
}

void MatmulLayer::clear_fusion() { fusion_.reset(); }
bool MatmulLayer::fused() const { return fusion_ != nullptr; }

// The weights are checked as in check(); the ends that stay plain rows are input 0 / output 0 of the layer, the
// other operands are checked by the kernel wrapper, like those of every GPU kernel of this API.
base::Status MatmulLayer::forward_fused() {
    const int32_t N = dim0_, K = dim1_, G = group_size_;
    if (G < 32 || G % 32 != 0 || K % G != 0 || N % 8 != 0) {
        return base::error::invalid_argument(
            "AWQ needs a group size that is a multiple of 32 and divides K, and N a multiple of 8.");
    }
    base::Status status = check_tensor_with_dim(get_weight(0), device_type_, base::DataType::DataTypeInt32, K, N / 8);
    if (status) status = check_tensor_with_dim(get_weight(1), device_type_, base::DataType::DataTypeInt32, K / G, N / 8);
    if (status) status = check_tensor_with_dim(scales_, device_type_, base::DataType::DataTypeFp16, K / G, N);
    if (!status) {
        LOG(ERROR) << "The weight tensor error in the matmul layer.";
        return status;
    }
    kernel::MatmulChain chain = *fusion_;
    if (chain.in == kernel::MatmulChain::In::Row) {
        chain.x = get_input(0);
        status = check_tensor(chain.x, device_type_, base::DataType::DataTypeBf16);
        if (status && batch_of(chain.x, K) != 1) status = base::error::invalid_argument("A fused launch takes one row [K].");
        if (!status) {
            LOG(ERROR) << "The input tensor error in the matmul layer.";
            return status;
        }
    }
    if (chain.out == kernel::MatmulChain::Out::Row) {
        chain.y = get_output(0);
        status = check_tensor(chain.y, device_type_, base::DataType::DataTypeBf16);
        if (status && batch_of(chain.y, N) != 1) status = base::error::invalid_argument("A fused launch writes one row [N].");
        if (!status) {
            LOG(ERROR) << "The output tensor error in the matmul layer.";
            return status;
        }
    }
    CHECK_NE(cuda_config_, nullptr);
    kernel::get_matmul_chain_kernel(device_type_)(chain, get_weight(0), scales_, get_weight(1), group_size_,
                                                  cuda_config_->stream());
    return base::error::success();
}

base::Status MatmulLayer::forward() {
    if (fusion_) {
        return forward_fused();
    }
    base::Status status = check();
    if (!status) {
        return status;
    }
    if (device_type_ == base::DeviceType::DeviceCUDA) {
        CHECK_NE(cuda_config_, nullptr);
    }
    void* stream = cuda_config_ ? cuda_config_->stream() : nullptr;
    if (is_quant_layer_) {
        kernel::get_matmul_kernel_awq(device_type_)(get_input(0), get_weight(0), scales_, get_weight(1),
                                                    get_output(0), group_size_, stream);
    } else {
        kernel::get_matmul_kernel(device_type_)(get_input(0), get_weight(0), get_output(0), stream);
    }
    return base::error::success();
}

}  // namespace op
