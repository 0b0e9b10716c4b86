// Qwen3-style decoder over the fused entry points of kx_hip.h (see model/qwen3_decoder.h).
#include "model/qwen3_decoder.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdlib>

#include "base/alloc.h"
#include "kernel/hip/matmul_kernel.h"
#include "kernel/kernel_interface.h"
#include "kx_hip.h"
#include "random_fill.h"

namespace model {
namespace {

constexpr int32_t kTileColumns = 256;          // columns per sum of squares that a residual launch leaves
constexpr int32_t kMergeInOMaxPositions = 10240;  // longest context the o projection can merge itself
constexpr int32_t kMergeInOMaxWorkgroups = 512;   // beyond this the separate merge launch is cheaper

std::string layer_prefix(int32_t i) { return "model.layers." + std::to_string(i) + "."; }

tensor::Tensor device_tensor(base::DataType type, const std::vector<int32_t>& dims) {
    tensor::Tensor t(type, dims, true, base::CUDADeviceAllocatorFactory::get_instance());
    CHECK_NE(t.ptr<uint8_t>(), nullptr);
    return t;
}

tensor::Tensor device_bytes(size_t bytes) {
    return device_tensor(base::DataType::DataTypeInt8, {static_cast<int32_t>(bytes)});
}

std::unique_ptr<op::MatmulLayer> awq_layer(int32_t n, int32_t k, int32_t group) {
    return std::make_unique<op::MatmulLayer>(base::DeviceType::DeviceCUDA, n, k, true, group);
}

uint16_t* u16(tensor::Tensor& t) { return t.ptr<uint16_t>(); }

struct Awq {
    const int32_t* qweight;
    const uint16_t* scales;
    const int32_t* qzeros;
};

Awq awq_of(const op::MatmulLayer& layer) {
    return Awq{layer.get_weight(0).ptr<int32_t>(), layer.awq_scales().ptr<uint16_t>(),
               layer.get_weight(1).ptr<int32_t>()};
}

bool metadata_number(const SafetensorsFile& file, const char* key, double& value) {
    auto it = file.metadata().find(key);
    if (it == file.metadata().end()) return false;
    char* end = nullptr;
    const double v = std::strtod(it->second.c_str(), &end);
    if (end == it->second.c_str()) return false;
    value = v;
    return true;
}

}  // namespace

base::Status Qwen3Config::from_file(const SafetensorsFile& file, Qwen3Config& config) {
    if (!file.is_open()) return base::error::invalid_argument("qwen3: the file is not open");
    Qwen3Config c;
    double number = 0.0;
    if (metadata_number(file, "rope_theta", number)) c.rope_theta = static_cast<float>(number);
    if (metadata_number(file, "rms_norm_eps", number)) c.rms_eps = static_cast<float>(number);
    if (metadata_number(file, "group_size", number)) c.group_size = static_cast<int32_t>(number);

    const TensorEntry* embed = file.find("model.embed_tokens.weight");
    if (!embed || embed->shape.size() != 2) {
        return base::error::model_parse_error("qwen3: model.embed_tokens.weight [vocab, hidden] is missing");
    }
    c.vocab = static_cast<int32_t>(embed->shape[0]);
    c.hidden = static_cast<int32_t>(embed->shape[1]);
    const std::string first = layer_prefix(0);
    const TensorEntry* q = file.find(first + "self_attn.q_proj.qweight");
    const TensorEntry* k = file.find(first + "self_attn.k_proj.qweight");
    const TensorEntry* gate = file.find(first + "mlp.gate_proj.qweight");
    if (!q || !k || !gate || q->shape.size() != 2 || k->shape.size() != 2 || gate->shape.size() != 2) {
        return base::error::model_parse_error("qwen3: q_proj / k_proj / gate_proj qweight of layer 0 are missing");
    }
    if ((q->shape[1] * 8) % c.head_dim || (k->shape[1] * 8) % c.head_dim) {
        return base::error::model_parse_error("qwen3: projection widths are not whole heads of 128");
    }
    c.n_q_heads = static_cast<int32_t>(q->shape[1] * 8 / c.head_dim);
    c.n_kv_heads = static_cast<int32_t>(k->shape[1] * 8 / c.head_dim);
    c.intermediate = static_cast<int32_t>(gate->shape[1] * 8);
    while (file.find(layer_prefix(c.layers) + "self_attn.q_proj.qweight") != nullptr) c.layers++;
    config = c;
    return base::error::success();
}

Qwen3Decoder::Qwen3Decoder(const Qwen3Config& config, int32_t max_positions, DecodePath path)
    : config_(config), max_positions_(max_positions), path_(path) {
    const Qwen3Config& c = config_;
    CHECK_EQ(c.head_dim, 128) << "the attention and rotary kernels are built for heads of 128";
    CHECK_GT(c.layers, 0);
    CHECK_GT(max_positions, 0);
    CHECK_GT(c.n_kv_heads, 0);
    CHECK_EQ(c.n_q_heads % c.n_kv_heads, 0);
    CHECK_EQ(c.hidden % 8, 0);
    CHECK_EQ(c.intermediate % 8, 0);

    stream_ = std::make_shared<kernel::CudaConfig>();
    stream_->create();

    // The o projection merges the attention chunks itself while it has about one round of
    // workgroups; with more, every one of them repeating the merge of its heads costs more than
    // the launch it saves.
    const int32_t o_workgroups =
        ((c.hidden + kTileColumns - 1) / kTileColumns) * std::max(1, c.n_q_heads * c.head_dim / kTileColumns);
    merge_in_o_ = max_positions <= kMergeInOMaxPositions && o_workgroups <= kMergeInOMaxWorkgroups;

    const base::DataType bf16 = base::DataType::DataTypeBf16;
    layers_.resize(static_cast<size_t>(c.layers));
    for (LayerWeights& L : layers_) {
        L.qkv = awq_layer(c.qkv_out(), c.hidden, c.group_size);
        L.o = awq_layer(c.hidden, c.n_q_heads * c.head_dim, c.group_size);
        L.gate_up = awq_layer(2 * c.intermediate, c.hidden, c.group_size);
        L.down = awq_layer(c.hidden, c.intermediate, c.group_size);
        L.k_cache = device_tensor(bf16, {max_positions, c.n_kv_heads, c.head_dim});
        L.v_cache = device_tensor(bf16, {max_positions, c.n_kv_heads, c.head_dim});
        // rows past the current position are read (and weighted with zero) by the attention kernel:
        // they must hold finite numbers
        CHECK_EQ(hipMemsetAsync(L.k_cache.ptr<uint8_t>(), 0, L.k_cache.byte_size(), stream()), hipSuccess);
        CHECK_EQ(hipMemsetAsync(L.v_cache.ptr<uint8_t>(), 0, L.v_cache.byte_size(), stream()), hipSuccess);
    }
    lm_head_ = std::make_unique<op::MatmulLayer>(base::DeviceType::DeviceCUDA, c.vocab, c.hidden, false);

    x_ = device_tensor(bf16, {c.hidden});
    h_ = device_tensor(bf16, {c.hidden});
    q_ = device_tensor(bf16, {c.n_q_heads * c.head_dim});
    attn_ = device_tensor(bf16, {c.n_q_heads * c.head_dim});
    gate_up_ = device_tensor(bf16, {2 * c.intermediate});
    logits_ = device_tensor(bf16, {c.vocab});
    // per 256 columns of the residual stream the sums of squares of its four quarters
    sumsq_ = device_tensor(base::DataType::DataTypeFp32, {(c.hidden + kTileColumns - 1) / kTileColumns, 4});
    io_ = device_tensor(base::DataType::DataTypeInt32, {3});

    const int32_t big_k = std::max(std::max(c.hidden, c.intermediate), c.n_q_heads * c.head_dim);
    const int32_t big_n = std::max(std::max(c.qkv_out(), 2 * c.intermediate), c.hidden);
    const size_t gemv_bytes = kx_gemv_workspace_bytes(1, big_k, big_n);
    CHECK_GT(gemv_bytes, 0u);
    gemv_workspace_ = device_bytes(gemv_bytes);
    CHECK_EQ(kx_workspace_init(gemv_workspace_.ptr<uint8_t>(), gemv_bytes, stream()), KX_OK);
    const size_t attn_bytes = kx_attn_decode_workspace_bytes(c.n_q_heads, c.head_dim, max_positions);
    CHECK_GT(attn_bytes, 0u) << "the attention kernels do not take this head layout or context length";
    attn_workspace_ = device_bytes(attn_bytes);

    CHECK_EQ(hipHostMalloc(reinterpret_cast<void**>(&host_io_), 3 * sizeof(int32_t), hipHostMallocDefault), hipSuccess);

    if (path_ != DecodePath::Fused) {
        const base::DeviceType gpu = base::DeviceType::DeviceCUDA;
        const bool operators = path_ == DecodePath::Operators;
        auto borrowed = [&](base::DataType type, int32_t n, void* ptr) {
            tensor::Tensor t(type, n, false, nullptr, ptr);
            t.set_device_type(gpu);  // a borrowed buffer does not know where it lives
            return t;
        };
        token_view_ = borrowed(base::DataType::DataTypeInt32, 1, io_.ptr<int32_t>());
        pos_view_ = borrowed(base::DataType::DataTypeInt32, 1, io_.ptr<int32_t>() + 1);
        gate_view_ = borrowed(bf16, c.intermediate, u16(gate_up_));
        up_view_ = borrowed(bf16, c.intermediate, u16(gate_up_) + c.intermediate);
        embedding_op_ = std::make_unique<op::EmbeddingLayer>(gpu, c.vocab, c.hidden);
        attention_op_ = std::make_unique<op::MultiHeadAttention>(gpu, c.n_q_heads, c.n_kv_heads);
        final_norm_op_ = std::make_unique<op::RmsNormLayer>(gpu, c.hidden, c.rms_eps);
        embedding_op_->set_cuda_config(stream_);
        attention_op_->set_cuda_config(stream_);
        final_norm_op_->set_cuda_config(stream_);
        lm_head_->set_cuda_config(stream_);
        if (operators) {
            qkv_ = device_tensor(bf16, {c.qkv_out()});
            o_ = device_tensor(bf16, {c.hidden});
            act_ = device_tensor(bf16, {c.intermediate});
            down_ = device_tensor(bf16, {c.hidden});
            swiglu_op_ = std::make_unique<op::SwiGLULayer>(gpu, c.intermediate);
            swiglu_op_->set_cuda_config(stream_);
        }
        // the fused path needs one stand-alone norm: the embedding row comes without its tile sums
        layer_ops_.resize(operators ? layers_.size() : 1);
        for (size_t i = 0; i < layer_ops_.size(); i++) {
            LayerOps& ops = layer_ops_[i];
            ops.input_norm = std::make_unique<op::RmsNormLayer>(gpu, c.hidden, c.rms_eps);
            ops.input_norm->set_cuda_config(stream_);
            if (!operators) continue;
            ops.post_norm = std::make_unique<op::RmsNormLayer>(gpu, c.hidden, c.rms_eps);
            ops.rope = std::make_unique<op::RoPELayer>(gpu, c.n_q_heads, c.n_kv_heads, c.rope_theta, c.rms_eps);
            ops.post_norm->set_cuda_config(stream_);
            ops.rope->set_cuda_config(stream_);
        }
        for (LayerWeights& L : layers_) {
            L.qkv->set_cuda_config(stream_);
            L.o->set_cuda_config(stream_);
            L.gate_up->set_cuda_config(stream_);
            L.down->set_cuda_config(stream_);
        }
        // everything a forward() would allocate on first use, now: a captured stream must not allocate
        CHECK(attention_op_->reserve(max_positions));
        kernel::matmul_reserve_workspace(stream(), 1, big_k, big_n);
    }
    CHECK_EQ(hipStreamSynchronize(stream()), hipSuccess);
}

Qwen3Decoder::~Qwen3Decoder() {
    if (stream_) (void)hipStreamSynchronize(stream());
    if (stream_ && path_ != DecodePath::Fused) kernel::matmul_release_workspace(stream());  // the stream goes away with us
    if (graph_exec_) (void)hipGraphExecDestroy(graph_exec_);
    if (graph_) (void)hipGraphDestroy(graph_);
    if (host_io_) (void)hipHostFree(host_io_);
}

base::Status Qwen3Decoder::load(const SafetensorsFile& file) {
    const Qwen3Config& c = config_;
    const base::DeviceType gpu = base::DeviceType::DeviceCUDA;
    base::Status st = load_bf16_tensor(file, "model.embed_tokens.weight", {c.vocab, c.hidden}, gpu, embed_);
    if (!st) return st;
    st = load_bf16_tensor(file, "model.norm.weight", {c.hidden}, gpu, final_norm_);
    if (!st) return st;
    if (file.find("lm_head.weight") != nullptr) {
        tensor::Tensor head;
        st = load_bf16_tensor(file, "lm_head.weight", {c.vocab, c.hidden}, gpu, head);
        if (!st) return st;
        st = lm_head_->set_weight(0, head);
    } else {
        st = lm_head_->set_weight(0, embed_);  // tied embeddings
    }
    if (!st) return st;
    for (int32_t i = 0; i < c.layers; i++) {
        LayerWeights& L = layers_[static_cast<size_t>(i)];
        const std::string p = layer_prefix(i);
        st = load_awq_linear_fused(file, {p + "self_attn.q_proj", p + "self_attn.k_proj", p + "self_attn.v_proj"}, *L.qkv);
        if (!st) return st;
        st = load_awq_linear(file, p + "self_attn.o_proj", *L.o);
        if (!st) return st;
        st = load_awq_linear_fused(file, {p + "mlp.gate_proj", p + "mlp.up_proj"}, *L.gate_up);
        if (!st) return st;
        st = load_awq_linear(file, p + "mlp.down_proj", *L.down);
        if (!st) return st;
        st = load_bf16_tensor(file, p + "input_layernorm.weight", {c.hidden}, gpu, L.input_norm);
        if (!st) return st;
        st = load_bf16_tensor(file, p + "post_attention_layernorm.weight", {c.hidden}, gpu, L.post_norm);
        if (!st) return st;
        st = load_bf16_tensor(file, p + "self_attn.q_norm.weight", {c.head_dim}, gpu, L.q_norm);
        if (!st) return st;
        st = load_bf16_tensor(file, p + "self_attn.k_norm.weight", {c.head_dim}, gpu, L.k_norm);
        if (!st) return st;
    }
    loaded_ = true;
    attach_layer_weights();
    return base::error::success();
}

void Qwen3Decoder::attach_layer_weights() {
    if (path_ == DecodePath::Fused) return;
    CHECK(embedding_op_->set_weight(0, embed_));
    CHECK(final_norm_op_->set_weight(0, final_norm_));
    if (path_ == DecodePath::Operators) {
        for (size_t i = 0; i < layers_.size(); i++) {
            CHECK(layer_ops_[i].input_norm->set_weight(0, layers_[i].input_norm));
            CHECK(layer_ops_[i].post_norm->set_weight(0, layers_[i].post_norm));
            CHECK(layer_ops_[i].rope->set_weight(0, layers_[i].q_norm));
            CHECK(layer_ops_[i].rope->set_weight(1, layers_[i].k_norm));
        }
        return;
    }
    // Layers: the fused form of every projection, set once; a step is then one forward() per launch
    const Qwen3Config& c = config_;
    using Chain = kernel::MatmulChain;
    CHECK(layer_ops_[0].input_norm->set_weight(0, layers_[0].input_norm));
    for (size_t i = 0; i < layers_.size(); i++) {
        LayerWeights& L = layers_[i];
        Chain qkv;
        if (i == 0) {
            qkv.in = Chain::In::Row;  // input 0 of the layer: the row the stand-alone norm leaves in h_
        } else {
            qkv.in = Chain::In::NormFromTileSums;
            qkv.norm_row = x_;
            qkv.norm_tile_sumsq = sumsq_;
            qkv.norm_gain = L.input_norm;
            qkv.norm_eps = c.rms_eps;
        }
        qkv.out = Chain::Out::QkvRope;
        qkv.q_gain = L.q_norm;
        qkv.k_gain = L.k_norm;
        qkv.q_out = q_;
        qkv.k_cache = L.k_cache;
        qkv.v_cache = L.v_cache;
        qkv.pos = pos_view_;
        qkv.rope_n_q_heads = c.n_q_heads;
        qkv.rope_n_kv_heads = c.n_kv_heads;
        qkv.rope_theta = c.rope_theta;
        qkv.qk_eps = c.rms_eps;
        CHECK(L.qkv->set_fusion(qkv));

        Chain o;
        if (merge_in_o_) {
            o.in = Chain::In::AttentionChunks;
            o.attention_chunks = attention_op_->chunks();  // reserved for max_positions in the constructor: it stays put
            o.n_q_heads = c.n_q_heads;
            o.n_kv_heads = c.n_kv_heads;
            o.max_positions = max_positions_;
        } else {
            o.in = Chain::In::Row;  // input 0: the merged attention output
        }
        o.out = Chain::Out::Residual;
        o.residual = x_;
        o.tile_sumsq = sumsq_;
        CHECK(L.o->set_fusion(o));

        Chain gate_up;
        gate_up.in = Chain::In::NormFromTileSums;
        gate_up.norm_row = x_;
        gate_up.norm_tile_sumsq = sumsq_;
        gate_up.norm_gain = L.post_norm;
        gate_up.norm_eps = c.rms_eps;
        gate_up.out = Chain::Out::Row;  // output 0 of the layer
        CHECK(L.gate_up->set_fusion(gate_up));

        Chain down;
        down.in = Chain::In::SwiGLU;
        down.gate = gate_view_;
        down.up = up_view_;
        down.out = Chain::Out::Residual;
        down.residual = x_;
        down.tile_sumsq = sumsq_;
        CHECK(L.down->set_fusion(down));
    }
}

void Qwen3Decoder::init_random(uint64_t seed) {
    const Qwen3Config& c = config_;
    void* s = stream();
    uint64_t stream_id = 0;
    auto next_seed = [&]() { return seed * 0x9E3779B97F4A7C15ull + (++stream_id << 40); };
    auto random_awq = [&](op::MatmulLayer& layer) {
        const int32_t N = layer.dim0(), K = layer.dim1(), G = layer.group_size();
        tensor::Tensor qweight = device_tensor(base::DataType::DataTypeInt32, {K, N / 8});
        tensor::Tensor qzeros = device_tensor(base::DataType::DataTypeInt32, {K / G, N / 8});
        tensor::Tensor scales = device_tensor(base::DataType::DataTypeFp16, {K / G, N});
        fill_random_words(qweight.ptr<int32_t>(), qweight.size(), next_seed(), s);
        fill_random_words(qzeros.ptr<int32_t>(), qzeros.size(), next_seed(), s);
        // |q - z| is about 4.6 on average: scales of 1 / (4.6 sqrt(K)) keep a row's magnitude
        const float unit = 1.0f / (4.6f * std::sqrt(static_cast<float>(K)));
        fill_uniform_fp16(scales.ptr<uint16_t>(), scales.size(), next_seed(), 0.75f * unit, 1.25f * unit, s);
        CHECK(layer.set_weight(0, qweight));
        CHECK(layer.set_weight(1, qzeros));
        layer.set_awq_scales(scales);
    };
    auto random_bf16 = [&](const std::vector<int32_t>& dims, float mean, float std) {
        tensor::Tensor t = device_tensor(base::DataType::DataTypeBf16, dims);
        fill_normal_bf16(t.ptr<uint16_t>(), t.size(), next_seed(), mean, std, s);
        return t;
    };
    for (LayerWeights& L : layers_) {
        random_awq(*L.qkv);
        random_awq(*L.o);
        random_awq(*L.gate_up);
        random_awq(*L.down);
        L.input_norm = random_bf16({c.hidden}, 1.0f, 0.02f);
        L.post_norm = random_bf16({c.hidden}, 1.0f, 0.02f);
        L.q_norm = random_bf16({c.head_dim}, 1.0f, 0.02f);
        L.k_norm = random_bf16({c.head_dim}, 1.0f, 0.02f);
    }
    embed_ = random_bf16({c.vocab, c.hidden}, 0.0f, 1.0f);
    final_norm_ = random_bf16({c.hidden}, 1.0f, 0.02f);
    CHECK(lm_head_->set_weight(0, random_bf16({c.vocab, c.hidden}, 0.0f, 0.02f)));
    CHECK_EQ(hipStreamSynchronize(stream()), hipSuccess);
    loaded_ = true;
    attach_layer_weights();
}

void Qwen3Decoder::fill_cache_random(int32_t positions, uint64_t seed) {
    CHECK_GE(positions, 0);
    CHECK_LE(positions, max_positions_);
    const size_t n = static_cast<size_t>(positions) * config_.n_kv_heads * config_.head_dim;
    uint64_t id = 0;
    for (LayerWeights& L : layers_) {
        fill_normal_bf16(u16(L.k_cache), n, seed * 0xD1342543DE82EF95ull + (++id << 40), 0.0f, 1.0f, stream());
        fill_normal_bf16(u16(L.v_cache), n, seed * 0xD1342543DE82EF95ull + (++id << 40), 0.0f, 1.0f, stream());
    }
    CHECK_EQ(hipStreamSynchronize(stream()), hipSuccess);
}

base::Status Qwen3Decoder::time_steps(int32_t token, int32_t pos, int32_t steps, int32_t warmup, double* ms_per_step) {
    if (!loaded_) return base::error::invalid_argument("qwen3: no weights");
    if (ms_per_step == nullptr || steps < 1 || warmup < 0) return base::error::invalid_argument("qwen3: bad arguments");
    int32_t next = 0;
    base::Status st = step(token, pos, &next);  // uploads token and position, checks them
    if (!st) return st;
    hipEvent_t begin = nullptr, end = nullptr;
    if (hipEventCreate(&begin) != hipSuccess || hipEventCreate(&end) != hipSuccess) {
        return base::error::internal_error("qwen3: event creation failed");
    }
    int rc = KX_OK;
    hipError_t err = hipSuccess;
    for (int32_t i = 0; i < warmup + steps && rc == KX_OK && err == hipSuccess; i++) {
        if (i == warmup) err = hipEventRecord(begin, stream());
        if (err != hipSuccess) break;
        if (graph_exec_) {
            err = hipGraphLaunch(graph_exec_, stream());
        } else {
            rc = enqueue_step();
        }
    }
    if (rc == KX_OK && err == hipSuccess) err = hipEventRecord(end, stream());
    const hipError_t sync = hipStreamSynchronize(stream());  // also after a failure: nothing may be left in flight
    float ms = 0.0f;
    if (rc == KX_OK && err == hipSuccess && sync == hipSuccess) err = hipEventElapsedTime(&ms, begin, end);
    (void)hipEventDestroy(begin);
    (void)hipEventDestroy(end);
    if (rc != KX_OK) return base::error::internal_error(std::string("qwen3: launch failed: ") + kx_error_string(rc));
    if (err != hipSuccess || sync != hipSuccess) {
        return base::error::internal_error(std::string("qwen3: timing: ") + hipGetErrorString(err != hipSuccess ? err : sync));
    }
    *ms_per_step = static_cast<double>(ms) / steps;
    return base::error::success();
}

int32_t Qwen3Decoder::launches_per_step() const {
    const int32_t per_layer = path_ == DecodePath::Operators ? 10 : (merge_in_o_ ? 5 : 6);
    // embedding; layers; final norm, lm_head, argmax; the Layers path norms the embedding row in a launch of its own
    return 1 + config_.layers * per_layer + 3 + (path_ == DecodePath::Layers ? 1 : 0);
}

int Qwen3Decoder::enqueue_step() {
    switch (path_) {
        case DecodePath::Layers: return enqueue_step_layers();
        case DecodePath::Operators: return enqueue_step_operators();
        default: return enqueue_step_fused();
    }
}

// One forward() per operator, in the order of the model's formulas.  A layer reports a refused
// tensor through its Status; a failed launch aborts inside the layer's kernel wrapper, as in the
// reference's GPU wrappers.
int Qwen3Decoder::enqueue_step_operators() {
    const Qwen3Config& c = config_;
#define KX_LAYER(call)                          \
    do {                                        \
        const base::Status layer_status = call; \
        if (!layer_status) {                    \
            LOG(ERROR) << layer_status.get_err_msg(); \
            return KX_ERR_BAD_SHAPE;            \
        }                                       \
    } while (0)
    KX_LAYER(embedding_op_->forward(token_view_, x_));
    for (int32_t li = 0; li < c.layers; li++) {
        LayerWeights& L = layers_[static_cast<size_t>(li)];
        LayerOps& ops = layer_ops_[static_cast<size_t>(li)];
        if (li == 0) {
            KX_LAYER(ops.input_norm->forward(x_, h_));
        } else {
            KX_LAYER(ops.input_norm->forward(x_, down_, h_));  // x += down of the previous layer, then the norm
        }
        KX_LAYER(L.qkv->forward(h_, qkv_));
        KX_LAYER(ops.rope->forward(qkv_, pos_view_, L.k_cache, L.v_cache, q_));
        KX_LAYER(attention_op_->forward(q_, pos_view_, L.k_cache, L.v_cache, attn_));
        KX_LAYER(L.o->forward(attn_, o_));
        KX_LAYER(ops.post_norm->forward(x_, o_, h_));
        KX_LAYER(L.gate_up->forward(h_, gate_up_));
        KX_LAYER(swiglu_op_->forward(gate_view_, up_view_, act_));
        KX_LAYER(L.down->forward(act_, down_));
    }
    KX_LAYER(final_norm_op_->forward(x_, down_, h_));
    KX_LAYER(lm_head_->forward(h_, logits_));
#undef KX_LAYER
    return kx_argmax_bf16(u16(logits_), c.vocab, io_.ptr<int32_t>() + 2, stream());
}

// The launches of enqueue_step_fused(), each as the forward() of a kuiper layer (the projections in their fused
// form, set in attach_layer_weights()).  The first layer's row is normed by a stand-alone RmsNormLayer: the
// embedding leaves no tile sums of squares for the fused form to start from.
int Qwen3Decoder::enqueue_step_layers() {
    const Qwen3Config& c = config_;
#define KX_LAYER(call)                          \
    do {                                        \
        const base::Status layer_status = call; \
        if (!layer_status) {                    \
            LOG(ERROR) << layer_status.get_err_msg(); \
            return KX_ERR_BAD_SHAPE;            \
        }                                       \
    } while (0)
    KX_LAYER(embedding_op_->forward(token_view_, x_));
    for (int32_t li = 0; li < c.layers; li++) {
        LayerWeights& L = layers_[static_cast<size_t>(li)];
        if (li == 0) {
            KX_LAYER(layer_ops_[0].input_norm->forward(x_, h_));
            L.qkv->set_input(0, h_);
        }
        KX_LAYER(L.qkv->forward());
        if (merge_in_o_) {
            KX_LAYER(attention_op_->forward_chunks(q_, pos_view_, L.k_cache, L.v_cache));
        } else {
            KX_LAYER(attention_op_->forward(q_, pos_view_, L.k_cache, L.v_cache, attn_));
            L.o->set_input(0, attn_);
        }
        KX_LAYER(L.o->forward());
        L.gate_up->set_output(0, gate_up_);
        KX_LAYER(L.gate_up->forward());
        KX_LAYER(L.down->forward());
    }
    KX_LAYER(final_norm_op_->forward(x_, h_));
    KX_LAYER(lm_head_->forward(h_, logits_));
#undef KX_LAYER
    return kx_argmax_bf16(u16(logits_), c.vocab, io_.ptr<int32_t>() + 2, stream());
}

int Qwen3Decoder::enqueue_step_fused() {
    const Qwen3Config& c = config_;
    void* s = stream();
    void* ws = gemv_workspace_.ptr<uint8_t>();
    const size_t ws_bytes = gemv_workspace_.byte_size();
    void* attn_ws = attn_workspace_.ptr<uint8_t>();
    const size_t attn_ws_bytes = attn_workspace_.byte_size();
    const int32_t* token = io_.ptr<int32_t>();
    const int32_t* pos = token + 1;
    int32_t* next = io_.ptr<int32_t>() + 2;
    const int32_t H = c.hidden, I = c.intermediate, QD = c.n_q_heads * c.head_dim, G = c.group_size;
    const int32_t parts = sumsq_.get_dim(0);

    int rc = kx_embedding_bf16(u16(embed_), token, u16(x_), c.vocab, H, s);
    if (rc != KX_OK) return rc;

    kx_chain_desc into_residual{};
    into_residual.out_kind = KX_OUT_RESIDUAL;
    into_residual.residual_in = u16(x_);
    into_residual.residual_out = u16(x_);
    into_residual.sumsq_out = sumsq_.ptr<float>();

    for (int32_t li = 0; li < c.layers; li++) {
        LayerWeights& L = layers_[static_cast<size_t>(li)];
        uint16_t* kc = u16(L.k_cache);
        uint16_t* vc = u16(L.v_cache);
        Awq w = awq_of(*L.qkv);
        if (li == 0) {
            // the embedding row arrives without its sums of squares: this launch norms the whole row itself
            rc = kx_gemv_awq_qkv_rope_bf16(u16(x_), nullptr, u16(L.input_norm), c.rms_eps, nullptr, w.qweight, w.scales,
                                           w.qzeros, u16(L.q_norm), u16(L.k_norm), u16(q_), kc, vc, c.n_q_heads,
                                           c.n_kv_heads, c.head_dim, pos, max_positions_, c.rope_theta, c.rms_eps, H,
                                           G, ws, ws_bytes, s);
        } else {
            kx_chain_desc d{};
            d.in_kind = KX_IN_NORM;
            d.norm_row = u16(x_);
            d.norm_sumsq = sumsq_.ptr<float>();
            d.norm_parts = parts;
            d.norm_gain = u16(L.input_norm);
            d.norm_eps = c.rms_eps;
            d.out_kind = KX_OUT_QKV_ROPE;
            d.q_gain = u16(L.q_norm);
            d.k_gain = u16(L.k_norm);
            d.q_out = u16(q_);
            d.k_cache = kc;
            d.v_cache = vc;
            d.pos = pos;
            d.rope_n_q_heads = c.n_q_heads;
            d.rope_n_kv_heads = c.n_kv_heads;
            d.cache_positions = max_positions_;
            d.rope_theta = c.rope_theta;
            d.qk_eps = c.rms_eps;
            rc = kx_gemv_awq_chain_bf16(&d, w.qweight, w.scales, w.qzeros, H, c.qkv_out(), G, ws, ws_bytes, s);
        }
        if (rc != KX_OK) return rc;

        w = awq_of(*L.o);
        kx_chain_desc o = into_residual;
        if (merge_in_o_) {
            rc = kx_attn_decode_partial_bf16(u16(q_), kc, vc, c.n_q_heads, c.n_kv_heads, c.head_dim, pos, max_positions_,
                                             attn_ws, attn_ws_bytes, s);
            o.in_kind = KX_IN_ATTN;
            o.attn_workspace = attn_ws;
            o.attn_workspace_bytes = attn_ws_bytes;
            o.n_q_heads = c.n_q_heads;
            o.n_kv_heads = c.n_kv_heads;
            o.max_positions = max_positions_;
        } else {
            rc = kx_attn_decode_bf16(u16(q_), kc, vc, u16(attn_), c.n_q_heads, c.n_kv_heads, c.head_dim, pos,
                                     max_positions_, attn_ws, attn_ws_bytes, s);
            o.in_kind = KX_IN_ROW;
            o.x = u16(attn_);
        }
        if (rc != KX_OK) return rc;
        rc = kx_gemv_awq_chain_bf16(&o, w.qweight, w.scales, w.qzeros, QD, H, G, ws, ws_bytes, s);
        if (rc != KX_OK) return rc;

        w = awq_of(*L.gate_up);
        kx_chain_desc gu{};
        gu.in_kind = KX_IN_NORM;
        gu.norm_row = u16(x_);
        gu.norm_sumsq = sumsq_.ptr<float>();
        gu.norm_parts = parts;
        gu.norm_gain = u16(L.post_norm);
        gu.norm_eps = c.rms_eps;
        gu.out_kind = KX_OUT_ROW;
        gu.y = u16(gate_up_);
        rc = kx_gemv_awq_chain_bf16(&gu, w.qweight, w.scales, w.qzeros, H, 2 * I, G, ws, ws_bytes, s);
        if (rc != KX_OK) return rc;

        w = awq_of(*L.down);
        kx_chain_desc down = into_residual;
        down.in_kind = KX_IN_SWIGLU;
        down.gate = u16(gate_up_);
        down.up = u16(gate_up_) + I;
        rc = kx_gemv_awq_chain_bf16(&down, w.qweight, w.scales, w.qzeros, I, H, G, ws, ws_bytes, s);
        if (rc != KX_OK) return rc;
    }

    rc = kx_rmsnorm_bf16(u16(x_), u16(final_norm_), u16(h_), 1, H, c.rms_eps, s);
    if (rc != KX_OK) return rc;
    rc = kx_gemv_bf16(u16(h_), lm_head_->get_weight(0).ptr<uint16_t>(), u16(logits_), 1, H, c.vocab, nullptr, 0, s);
    if (rc != KX_OK) return rc;
    return kx_argmax_bf16(u16(logits_), c.vocab, next, s);
}

base::Status Qwen3Decoder::capture() {
    if (!loaded_) return base::error::invalid_argument("qwen3: load() the weights before capture()");
    if (graph_exec_) return base::error::success();
    hipError_t err = hipStreamBeginCapture(stream(), hipStreamCaptureModeThreadLocal);
    if (err != hipSuccess) return base::error::internal_error(std::string("qwen3: begin capture: ") + hipGetErrorString(err));
    const int rc = enqueue_step();
    err = hipStreamEndCapture(stream(), &graph_);  // always end the capture, also after a failed launch
    if (rc != KX_OK) {
        if (graph_) (void)hipGraphDestroy(graph_);
        graph_ = nullptr;
        return base::error::internal_error(std::string("qwen3: a launch failed during capture: ") + kx_error_string(rc));
    }
    if (err != hipSuccess) return base::error::internal_error(std::string("qwen3: end capture: ") + hipGetErrorString(err));
    err = hipGraphInstantiate(&graph_exec_, graph_, nullptr, nullptr, 0);
    if (err != hipSuccess) {
        graph_exec_ = nullptr;
        return base::error::internal_error(std::string("qwen3: instantiate: ") + hipGetErrorString(err));
    }
    return base::error::success();
}

base::Status Qwen3Decoder::step(int32_t token, int32_t pos, int32_t* next_token) {
    if (!loaded_) return base::error::invalid_argument("qwen3: load() the weights before step()");
    if (next_token == nullptr) return base::error::invalid_argument("qwen3: next_token is null");
    if (token < 0 || token >= config_.vocab) return base::error::invalid_argument("qwen3: token outside the vocabulary");
    if (pos < 0 || pos >= max_positions_) return base::error::invalid_argument("qwen3: position outside the caches");
    host_io_[0] = token;
    host_io_[1] = pos;
    hipError_t err = hipMemcpyAsync(io_.ptr<int32_t>(), host_io_, 2 * sizeof(int32_t), hipMemcpyHostToDevice, stream());
    if (err != hipSuccess) return base::error::internal_error(std::string("qwen3: upload: ") + hipGetErrorString(err));
    if (graph_exec_) {
        err = hipGraphLaunch(graph_exec_, stream());
        if (err != hipSuccess) return base::error::internal_error(std::string("qwen3: graph launch: ") + hipGetErrorString(err));
    } else {
        const int rc = enqueue_step();
        if (rc != KX_OK) return base::error::internal_error(std::string("qwen3: launch failed: ") + kx_error_string(rc));
    }
    err = hipMemcpyAsync(host_io_ + 2, io_.ptr<int32_t>() + 2, sizeof(int32_t), hipMemcpyDeviceToHost, stream());
    if (err == hipSuccess) err = hipStreamSynchronize(stream());
    if (err != hipSuccess) return base::error::internal_error(std::string("qwen3: step: ") + hipGetErrorString(err));
    *next_token = host_io_[2];
    return base::error::success();
}

std::vector<uint16_t> Qwen3Decoder::logits() const {
    std::vector<uint16_t> host(static_cast<size_t>(config_.vocab));
    CHECK_EQ(hipStreamSynchronize(stream()), hipSuccess);
    CHECK_EQ(hipMemcpy(host.data(), logits_.ptr<uint16_t>(), host.size() * sizeof(uint16_t), hipMemcpyDeviceToHost),
             hipSuccess);
    return host;
}

}  // namespace model
