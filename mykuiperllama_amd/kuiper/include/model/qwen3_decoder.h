// Qwen3-style decoder, one token at a time (batch 1), on the GPU: INT4 AWQ projections, bf16 KV
// cache, greedy sampling.  The reference lists kuiper/source/model/ in its build
// (CMakeLists.txt:79) and the directory is absent; the layer slots of kuiper/include/op/layer.h:8-20
// say which operators a model is made of.  This is the runner for them: weights attach through
// MatmulLayer (model/safetensors.h), and a step is the launch sequence of include/kx_hip.h's fused
// entry points, five or six launches per decoder layer:
//
//   x = embed[token]
//   per layer:  q|k|v GEMV   (RMSNorm on the way in; per-head norm, rotation, cache append on the way out)
//               attention    (partial results per chunk of the context)
//               o GEMV       (merge of the chunks on the way in when the context allows; residual add out)
//               gate|up GEMV (RMSNorm on the way in)
//               down GEMV    (SwiGLU on the way in; residual add out)
//   logits = lm_head RMSNorm(x);  next = argmax(logits)
//
// Token and position are read from device memory, so the whole step can be captured once in a HIP
// graph and replayed for every token: capture() does that, step() then replays.
#ifndef KUIPER_INCLUDE_MODEL_QWEN3_DECODER_H
#define KUIPER_INCLUDE_MODEL_QWEN3_DECODER_H

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "base/base.h"
#include "base/cuda_config.h"
#include "model/safetensors.h"
#include "op/embedding.h"
#include "op/matmul.h"
#include "op/mha.h"
#include "op/rmsnorm.h"
#include "op/rope.h"
#include "op/swiglu.h"
#include "tensor/tensor.h"

namespace model {

struct Qwen3Config {
    int32_t layers = 0;
    int32_t hidden = 0;
    int32_t intermediate = 0;
    int32_t n_q_heads = 0;
    int32_t n_kv_heads = 0;
    int32_t vocab = 0;
    int32_t head_dim = 128;  // the only head size the kernels are built for
    int32_t group_size = 128;
    float rope_theta = 1e6f;
    float rms_eps = 1e-6f;

    int32_t qkv_out() const { return (n_q_heads + 2 * n_kv_heads) * head_dim; }

    // Reads the sizes off the tensors of a checkpoint with Hugging Face's Qwen3 names
    // (model.layers.<i>.self_attn.q_proj.qweight ...).  rope_theta / rms_norm_eps / group_size are
    // taken from the file's metadata when present.
    static base::Status from_file(const SafetensorsFile& file, Qwen3Config& config);
};

// How a step is put together.
//   Fused      the fused entry points of kx_hip.h called directly, five or six launches per decoder layer
//   Layers     the same launches through the layer API of kuiper/include/op/layer.h: every launch is the
//              forward() of a kuiper layer — EmbeddingLayer, RmsNormLayer (first layer's input and the final norm),
//              MultiHeadAttention (its first stage), and four MatmulLayers per decoder layer whose fused form
//              (MatmulLayer::set_fusion) carries the norms, the rotation, the merge, SwiGLU and the residual add
//   Operators  one kuiper layer per operator, forward() by forward() — EmbeddingLayer, RmsNormLayer (with
//              the residual add in front), MatmulLayer, RoPELayer, MultiHeadAttention, SwiGLULayer — ten
//              launches per decoder layer: a model that uses the layer API without the fused forms, and the
//              yardstick the other two are held against
enum class DecodePath { Fused, Layers, Operators };

class Qwen3Decoder {
public:
    // Allocates caches and scratch rows for max_positions positions.  The decoder runs on a stream
    // of its own (graph capture needs one that is not the default stream).
    Qwen3Decoder(const Qwen3Config& config, int32_t max_positions, DecodePath path = DecodePath::Fused);
    ~Qwen3Decoder();
    Qwen3Decoder(const Qwen3Decoder&) = delete;
    Qwen3Decoder& operator=(const Qwen3Decoder&) = delete;

    // Copies the weights to the GPU: q|k|v and gate|up side by side along N, norms, embedding,
    // lm_head (the embedding table when the file has no lm_head.weight).  BF16 or F16 on file for the
    // unquantised tensors (F16 is rounded to bf16).
    base::Status load(const SafetensorsFile& file);

    // Random-init weights of the configured architecture instead of a checkpoint (benchmarks): packed
    // words uniform, scales sized so that activations keep O(1) magnitude through the layers, norm
    // gains 1 + 0.02 N(0,1), embedding N(0,1), lm_head 0.02 N(0,1).  Seeded; nothing is read from disk.
    void init_random(uint64_t seed);
    // Rows 0 .. positions-1 of every cache set to bf16 N(0,1), the state a benchmark decodes from.
    void fill_cache_random(int32_t positions, uint64_t seed);

    // One token at position pos (0 <= pos < max_positions): appends its key and value to the caches
    // and returns the most likely next token.  Synchronises the decoder's stream.
    base::Status step(int32_t token, int32_t pos, int32_t* next_token);

    // Records the step in a HIP graph; later step() calls replay it.
    base::Status capture();
    bool captured() const { return graph_exec_ != nullptr; }

    // `steps` steps of the same token at the same position back to back (after `warmup` untimed
    // ones), timed with events on the decoder's stream; replays the graph when one is captured.
    base::Status time_steps(int32_t token, int32_t pos, int32_t steps, int32_t warmup, double* ms_per_step);

    // bf16 logits of the last step, copied to the host.
    std::vector<uint16_t> logits() const;

    const Qwen3Config& config() const { return config_; }
    DecodePath path() const { return path_; }
    int32_t max_positions() const { return max_positions_; }
    int32_t launches_per_step() const;
    hipStream_t stream() const { return stream_->stream(); }

private:
    struct LayerWeights {
        std::unique_ptr<op::MatmulLayer> qkv, o, gate_up, down;
        tensor::Tensor input_norm, post_norm, q_norm, k_norm;
        tensor::Tensor k_cache, v_cache;
    };

    struct LayerOps {
        std::unique_ptr<op::RmsNormLayer> input_norm, post_norm;
        std::unique_ptr<op::RoPELayer> rope;
    };

    int enqueue_step();  // 0 or the first failing entry point's return code
    int enqueue_step_fused();
    int enqueue_step_layers();
    int enqueue_step_operators();
    void attach_layer_weights();  // Layers and Operators paths: gains and tables into the layers, fused forms set

    Qwen3Config config_;
    int32_t max_positions_ = 0;
    DecodePath path_ = DecodePath::Fused;
    bool merge_in_o_ = false;
    bool loaded_ = false;
    std::shared_ptr<kernel::CudaConfig> stream_;
    std::vector<LayerWeights> layers_;
    tensor::Tensor embed_, final_norm_;
    std::unique_ptr<op::MatmulLayer> lm_head_;
    tensor::Tensor x_, h_, q_, attn_, gate_up_, logits_, sumsq_;
    // Layers and Operators paths
    std::vector<LayerOps> layer_ops_;
    std::unique_ptr<op::EmbeddingLayer> embedding_op_;
    std::unique_ptr<op::MultiHeadAttention> attention_op_;
    std::unique_ptr<op::SwiGLULayer> swiglu_op_;
    std::unique_ptr<op::RmsNormLayer> final_norm_op_;
    tensor::Tensor qkv_, o_, act_, down_;
    tensor::Tensor token_view_, pos_view_, gate_view_, up_view_;  // borrowed pieces of io_ and gate_up_
    tensor::Tensor gemv_workspace_, attn_workspace_;
    tensor::Tensor io_;           // device: token, position, next token (int32 each)
    int32_t* host_io_ = nullptr;  // pinned mirror of io_
    hipGraph_t graph_ = nullptr;
    hipGraphExec_t graph_exec_ = nullptr;
};

}  // namespace model

#endif  // KUIPER_INCLUDE_MODEL_QWEN3_DECODER_H
