// The decode-step operator layers: shape checks and dispatch, in the structure of the reference's one
// concrete layer (kuiper/source/op/add.cpp:5-49): check(), then the kernel of the layer's device on
// the layer's stream.
#include <string>

#include <hip/hip_runtime_api.h>

#include "kernel/kernel_interface.h"
#include "kx_hip.h"
#include "op/embedding.h"
#include "op/mha.h"
#include "op/rmsnorm.h"
#include "op/rope.h"
#include "op/swiglu.h"

namespace op {
namespace {
constexpr int32_t kHeadDim = 128;
}

// ---------------------------------------------------------------- TypedLayer
TypedLayer::TypedLayer(base::DeviceType device_type, LayerType layer_type, std::string layer_name)
    : LayerParam(device_type, layer_type, false, std::move(layer_name)) {
    data_type_ = base::DataType::DataTypeBf16;
}

void TypedLayer::set_input(int32_t idx, const tensor::Tensor& input) {
    CHECK_GE(idx, 0);
    CHECK_LT(static_cast<size_t>(idx), inputs_.size());
    if (!input.is_empty()) {
        CHECK(input.device_type() == device_type_);
    }
    inputs_[idx] = input;
}

void TypedLayer::set_output(int32_t idx, const tensor::Tensor& output) {
    CHECK_GE(idx, 0);
    CHECK_LT(static_cast<size_t>(idx), outputs_.size());
    if (!output.is_empty()) {
        CHECK(output.device_type() == device_type_);
    }
    outputs_[idx] = output;
}

base::Status TypedLayer::set_weight(int32_t idx, const tensor::Tensor& weight) {
    CHECK_GE(idx, 0);
    CHECK_LT(static_cast<size_t>(idx), weights_.size());
    CHECK(weight.data_type() == base::DataType::DataTypeBf16);
    if (!weight.is_empty()) {
        CHECK(weight.device_type() == device_type_);
    }
    weights_[idx] = weight;
    return base::error::success();
}

void* TypedLayer::stream() const {
    return cuda_config_ ? cuda_config_->stream() : nullptr;
}

base::Status TypedLayer::expect(const tensor::Tensor& t, base::DataType type, size_t elements,
                                const char* what) const {
    if (t.is_empty()) {
        return base::error::invalid_argument(std::string("The ") + what + " tensor of the " + layer_name_ + " layer is empty.");
    }
    if (t.device_type() != device_type_) {
        return base::error::invalid_argument(std::string("The ") + what + " tensor has a wrong device type.");
    }
    if (t.data_type() != type) {
        return base::error::invalid_argument(std::string("The ") + what + " tensor has a wrong data type.");
    }
    if (t.size() != elements) {
        return base::error::invalid_argument(std::string("The ") + what + " tensor has a wrong size.");
    }
    return base::error::success();
}

#define KX_RETURN_IF_BAD(call)          \
    do {                                \
        const base::Status st_ = call;  \
        if (!st_) {                     \
            LOG(ERROR) << st_;          \
            return st_;                 \
        }                               \
    } while (0)

// ---------------------------------------------------------------- RmsNormLayer
RmsNormLayer::RmsNormLayer(base::DeviceType device_type, int32_t dim, float eps)
    : TypedLayer(device_type, LayerType::LayerRMSNorm, "RMSNorm"), dim_(dim), eps_(eps) {
    reset_input_size(2);
    reset_output_size(1);
    reset_weights_size(1);
}

base::Status RmsNormLayer::check() const {
    const tensor::Tensor& x = get_input(0);
    if (x.is_empty() || dim_ <= 0 || x.size() % static_cast<size_t>(dim_) != 0 ||
        x.get_dim(x.dims_size() - 1) != dim_) {
        return base::error::invalid_argument("The input tensor error in the rmsnorm layer.");
    }
    KX_RETURN_IF_BAD(expect(x, base::DataType::DataTypeBf16, x.size(), "input"));
    if (!get_input(1).is_empty()) {
        KX_RETURN_IF_BAD(expect(get_input(1), base::DataType::DataTypeBf16, x.size(), "delta"));
    }
    KX_RETURN_IF_BAD(expect(get_weight(0), base::DataType::DataTypeBf16, static_cast<size_t>(dim_), "gain"));
    KX_RETURN_IF_BAD(expect(get_output(0), base::DataType::DataTypeBf16, x.size(), "output"));
    return base::error::success();
}

base::Status RmsNormLayer::forward() {
    const base::Status status = check();
    if (!status) return status;
    kernel::get_rmsnorm_kernel(device_type_)(get_input(0), get_input(1), get_weight(0), get_output(0), eps_, stream());
    return base::error::success();
}

// ---------------------------------------------------------------- SwiGLULayer
SwiGLULayer::SwiGLULayer(base::DeviceType device_type, int32_t dim)
    : TypedLayer(device_type, LayerType::LayerSwiGLU, "SwiGLU"), dim_(dim) {
    reset_input_size(2);
    reset_output_size(1);
}

base::Status SwiGLULayer::check() const {
    const size_t n = static_cast<size_t>(dim_);
    KX_RETURN_IF_BAD(expect(get_input(0), base::DataType::DataTypeBf16, n, "gate"));
    KX_RETURN_IF_BAD(expect(get_input(1), base::DataType::DataTypeBf16, n, "up"));
    KX_RETURN_IF_BAD(expect(get_output(0), base::DataType::DataTypeBf16, n, "output"));
    return base::error::success();
}

base::Status SwiGLULayer::forward() {
    const base::Status status = check();
    if (!status) return status;
    kernel::get_swiglu_kernel(device_type_)(get_input(0), get_input(1), get_output(0), stream());
    return base::error::success();
}

// ---------------------------------------------------------------- EmbeddingLayer
EmbeddingLayer::EmbeddingLayer(base::DeviceType device_type, int32_t vocab, int32_t dim)
    : TypedLayer(device_type, LayerType::LayerEmbedding, "Embedding"), vocab_(vocab), dim_(dim) {
    reset_input_size(1);
    reset_output_size(1);
    reset_weights_size(1);
}

base::Status EmbeddingLayer::check() const {
    KX_RETURN_IF_BAD(expect(get_input(0), base::DataType::DataTypeInt32, 1, "token"));
    KX_RETURN_IF_BAD(expect(get_weight(0), base::DataType::DataTypeBf16, static_cast<size_t>(vocab_) * dim_, "table"));
    if (get_weight(0).dims_size() != 2 || get_weight(0).get_dim(0) != vocab_) {
        return base::error::invalid_argument("The embedding table must be [vocab, dim].");
    }
    KX_RETURN_IF_BAD(expect(get_output(0), base::DataType::DataTypeBf16, static_cast<size_t>(dim_), "output"));
    return base::error::success();
}

base::Status EmbeddingLayer::forward() {
    const base::Status status = check();
    if (!status) return status;
    kernel::get_embedding_kernel(device_type_)(get_input(0), get_weight(0), get_output(0), stream());
    return base::error::success();
}

// ---------------------------------------------------------------- RoPELayer
RoPELayer::RoPELayer(base::DeviceType device_type, int32_t n_q_heads, int32_t n_kv_heads, float theta, float eps)
    : TypedLayer(device_type, LayerType::LayerRope, "RoPE"), n_q_(n_q_heads), n_kv_(n_kv_heads), theta_(theta), eps_(eps) {
    reset_input_size(4);
    reset_output_size(1);
    reset_weights_size(2);
}

base::Status RoPELayer::check() const {
    if (n_q_ < 1 || n_kv_ < 1 || !(theta_ > 1.0f)) {
        return base::error::invalid_argument("The head counts or theta of the rope layer are invalid.");
    }
    KX_RETURN_IF_BAD(expect(get_input(0), base::DataType::DataTypeBf16, static_cast<size_t>(n_q_ + 2 * n_kv_) * kHeadDim, "qkv"));
    KX_RETURN_IF_BAD(expect(get_input(1), base::DataType::DataTypeInt32, 1, "pos"));
    const tensor::Tensor& kc = get_input(2);
    if (kc.is_empty() || kc.dims_size() != 3 || kc.get_dim(1) != n_kv_ || kc.get_dim(2) != kHeadDim) {
        return base::error::invalid_argument("The key cache must be [max_positions, n_kv_heads, 128].");
    }
    KX_RETURN_IF_BAD(expect(kc, base::DataType::DataTypeBf16, kc.size(), "key cache"));
    KX_RETURN_IF_BAD(expect(get_input(3), base::DataType::DataTypeBf16, kc.size(), "value cache"));
    KX_RETURN_IF_BAD(expect(get_weight(0), base::DataType::DataTypeBf16, kHeadDim, "q gain"));
    KX_RETURN_IF_BAD(expect(get_weight(1), base::DataType::DataTypeBf16, kHeadDim, "k gain"));
    KX_RETURN_IF_BAD(expect(get_output(0), base::DataType::DataTypeBf16, static_cast<size_t>(n_q_) * kHeadDim, "q output"));
    return base::error::success();
}

base::Status RoPELayer::forward() {
    const base::Status status = check();
    if (!status) return status;
    kernel::get_rope_kernel(device_type_)(get_input(0), get_weight(0), get_weight(1), get_input(1), get_output(0),
                                          get_input(2), get_input(3), n_q_, n_kv_, theta_, eps_, stream());
    return base::error::success();
}

// ---------------------------------------------------------------- MultiHeadAttention
MultiHeadAttention::MultiHeadAttention(base::DeviceType device_type, int32_t n_q_heads, int32_t n_kv_heads)
    : TypedLayer(device_type, LayerType::LayerMHA, "MHA"), n_q_(n_q_heads), n_kv_(n_kv_heads) {
    reset_input_size(4);
    reset_output_size(1);
}

base::Status MultiHeadAttention::check() const {
    if (n_q_ < 1 || n_kv_ < 1 || n_q_ % n_kv_ != 0) {
        return base::error::invalid_argument("The head counts of the mha layer are invalid.");
    }
    const int32_t g = n_q_ / n_kv_;
    if (g > 16) {
        return base::error::invalid_argument("The mha layer serves up to 16 query heads per key/value head.");
    }
    KX_RETURN_IF_BAD(expect(get_input(0), base::DataType::DataTypeBf16, static_cast<size_t>(n_q_) * kHeadDim, "query"));
    KX_RETURN_IF_BAD(expect(get_input(1), base::DataType::DataTypeInt32, 1, "pos"));
    const tensor::Tensor& kc = get_input(2);
    if (kc.is_empty() || kc.dims_size() != 3 || kc.get_dim(1) != n_kv_ || kc.get_dim(2) != kHeadDim ||
        kc.get_dim(0) > 65536) {
        return base::error::invalid_argument("The key cache must be [max_positions <= 65536, n_kv_heads, 128].");
    }
    KX_RETURN_IF_BAD(expect(kc, base::DataType::DataTypeBf16, kc.size(), "key cache"));
    KX_RETURN_IF_BAD(expect(get_input(3), base::DataType::DataTypeBf16, kc.size(), "value cache"));
    KX_RETURN_IF_BAD(expect(get_output(0), base::DataType::DataTypeBf16, static_cast<size_t>(n_q_) * kHeadDim, "output"));
    return base::error::success();
}

// Makes the attention workspace at least `need` bytes.  The block it replaces may still be read and
// written by launches already enqueued on the layer's stream, and the allocator's pool would hand it
// out again at once, so the stream is drained first; while the stream records a graph neither that wait
// nor the allocation is possible, and the caller has to have reserved beforehand.
base::Status MultiHeadAttention::grow_workspace(size_t need) {
    if (!workspace_.is_empty() && workspace_.byte_size() >= need) return base::error::success();
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(static_cast<hipStream_t>(stream()), &capture) != hipSuccess) {
        (void)hipGetLastError();
        capture = hipStreamCaptureStatusNone;
    }
    if (capture != hipStreamCaptureStatusNone) {
        return base::error::invalid_argument(
            "mha: the attention workspace must grow while the stream is capturing; call reserve(max_positions) "
            "before the capture begins");
    }
    if (!workspace_.is_empty()) (void)hipStreamSynchronize(static_cast<hipStream_t>(stream()));
    workspace_ = tensor::Tensor(base::DataType::DataTypeInt8, static_cast<int32_t>(need), true,
                                base::CUDADeviceAllocatorFactory::get_instance());
    return base::error::success();
}

base::Status MultiHeadAttention::forward() {
    const base::Status status = check();
    if (!status) return status;
    if (device_type_ == base::DeviceType::DeviceCUDA) {
        const base::Status grown = grow_workspace(kx_attn_decode_workspace_bytes(n_q_, kHeadDim, get_input(2).get_dim(0)));
        if (!grown) return grown;
    }
    kernel::get_mha_kernel(device_type_)(get_input(0), get_input(2), get_input(3), get_input(1), workspace_,
                                         get_output(0), n_q_, n_kv_, stream());
    return base::error::success();
}

base::Status MultiHeadAttention::forward_chunks(const tensor::Tensor& q, const tensor::Tensor& pos,
                                                const tensor::Tensor& k_cache, const tensor::Tensor& v_cache) {
    if (device_type_ != base::DeviceType::DeviceCUDA) {
        return base::error::invalid_argument("mha: the unmerged chunks exist on the GPU only");
    }
    set_input(0, q);
    set_input(1, pos);
    set_input(2, k_cache);
    set_input(3, v_cache);
    // everything check() asks of the inputs; there is no output tensor in this form
    if (n_q_ < 1 || n_kv_ < 1 || n_q_ % n_kv_ != 0 || n_q_ / n_kv_ > 16) {
        return base::error::invalid_argument("The head counts of the mha layer are invalid.");
    }
    KX_RETURN_IF_BAD(expect(q, base::DataType::DataTypeBf16, static_cast<size_t>(n_q_) * kHeadDim, "query"));
    KX_RETURN_IF_BAD(expect(pos, base::DataType::DataTypeInt32, 1, "pos"));
    if (k_cache.is_empty() || k_cache.dims_size() != 3 || k_cache.get_dim(1) != n_kv_ || k_cache.get_dim(2) != kHeadDim ||
        k_cache.get_dim(0) > 65536) {
        return base::error::invalid_argument("The key cache must be [max_positions <= 65536, n_kv_heads, 128].");
    }
    KX_RETURN_IF_BAD(expect(k_cache, base::DataType::DataTypeBf16, k_cache.size(), "key cache"));
    KX_RETURN_IF_BAD(expect(v_cache, base::DataType::DataTypeBf16, k_cache.size(), "value cache"));
    const base::Status grown = grow_workspace(kx_attn_decode_workspace_bytes(n_q_, kHeadDim, k_cache.get_dim(0)));
    if (!grown) return grown;
    kernel::get_mha_kernel(device_type_)(q, k_cache, v_cache, pos, workspace_, tensor::Tensor(), n_q_, n_kv_, stream());
    return base::error::success();
}

base::Status MultiHeadAttention::reserve(int32_t max_positions) {
    if (device_type_ != base::DeviceType::DeviceCUDA) return base::error::success();
    const size_t need = kx_attn_decode_workspace_bytes(n_q_, kHeadDim, max_positions);
    if (need == 0) return base::error::invalid_argument("mha: no attention kernel for this head layout or context length");
    return grow_workspace(need);
}

#undef KX_RETURN_IF_BAD

}  // namespace op
