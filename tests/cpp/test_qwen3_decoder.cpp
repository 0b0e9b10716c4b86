// model::Qwen3Config / Qwen3Decoder (model/qwen3_decoder.h) and the bf16 tensor loader: what the
// runner reads off a checkpoint, what it refuses, and that a step replayed from the captured graph
// is the step enqueued launch by launch.  (That the step itself is right is checked from Python,
// bit for bit against the driver that is compared with an fp32 reference.)
#include <hip/hip_runtime_api.h>

#include <cstring>
#include <string>
#include <vector>

#include "../../oracle/kx_oracle.h"
#include "../../mykuiperllama_amd/kuiper/source/op/kernel/kernel_interface.h"
#include "mini_test.h"
#include "model/qwen3_decoder.h"
#include "model/safetensors.h"
#include "safetensors_writer.h"

namespace {

using namespace stw;

model::Qwen3Config tiny_config() {
    model::Qwen3Config c;
    c.layers = 2;
    c.hidden = 512;
    c.intermediate = 1024;
    c.n_q_heads = 4;
    c.n_kv_heads = 2;
    c.vocab = 1024;
    return c;
}

// only what Qwen3Config::from_file looks at: shapes, no meaningful values
void add_projection(std::vector<Blob>& blobs, const std::string& prefix, int K, int N) {
    blobs.push_back(blob(prefix + ".qweight", "I32", {K, N / 8}, std::vector<int32_t>(size_t(K) * N / 8, 0)));
}

std::vector<Blob> skeleton(int layers, int hidden, int q_width, int kv_width, int intermediate, int vocab) {
    std::vector<Blob> blobs;
    blobs.push_back(blob("model.embed_tokens.weight", "BF16", {vocab, hidden}, std::vector<uint16_t>(size_t(vocab) * hidden, 0)));
    for (int i = 0; i < layers; i++) {
        const std::string p = "model.layers." + std::to_string(i) + ".";
        add_projection(blobs, p + "self_attn.q_proj", hidden, q_width);
        add_projection(blobs, p + "self_attn.k_proj", hidden, kv_width);
        add_projection(blobs, p + "mlp.gate_proj", hidden, intermediate);
    }
    return blobs;
}

}  // namespace

TEST_CPU(test_qwen3_decoder, config_is_read_off_the_tensors) {
    TempFile tmp;
    tmp.write(serialise(skeleton(3, 256, 1024, 256, 768, 64),
                        "{\"rope_theta\":\"500000\",\"rms_norm_eps\":\"1e-5\",\"group_size\":\"64\",\"note\":\"x\"}"));
    model::SafetensorsFile file;
    ASSERT_TRUE(bool(file.open(tmp.path)));
    model::Qwen3Config c;
    ASSERT_TRUE(bool(model::Qwen3Config::from_file(file, c)));
    ASSERT_EQ(c.layers, 3);
    ASSERT_EQ(c.hidden, 256);
    ASSERT_EQ(c.vocab, 64);
    ASSERT_EQ(c.n_q_heads, 8);
    ASSERT_EQ(c.n_kv_heads, 2);
    ASSERT_EQ(c.intermediate, 768);
    ASSERT_EQ(c.qkv_out(), (8 + 2 * 2) * 128);
    ASSERT_EQ(c.group_size, 64);
    ASSERT_EQ(c.rope_theta, 500000.0f);
    ASSERT_EQ(c.rms_eps, 1e-5f);
}

TEST_CPU(test_qwen3_decoder, config_defaults_without_metadata) {
    TempFile tmp;
    tmp.write(serialise(skeleton(1, 256, 256, 128, 512, 32)));
    model::SafetensorsFile file;
    ASSERT_TRUE(bool(file.open(tmp.path)));
    model::Qwen3Config c;
    ASSERT_TRUE(bool(model::Qwen3Config::from_file(file, c)));
    ASSERT_EQ(c.layers, 1);
    ASSERT_EQ(c.group_size, 128);
    ASSERT_EQ(c.rope_theta, 1e6f);
    ASSERT_EQ(c.rms_eps, 1e-6f);
}

TEST_CPU(test_qwen3_decoder, config_refuses_files_that_hold_no_model) {
    model::Qwen3Config c;
    model::SafetensorsFile closed;
    ASSERT_FALSE(bool(model::Qwen3Config::from_file(closed, c)));
    {
        TempFile tmp;  // no embedding table
        std::vector<Blob> blobs = skeleton(1, 256, 256, 128, 512, 32);
        blobs.erase(blobs.begin());
        tmp.write(serialise(blobs));
        model::SafetensorsFile file;
        ASSERT_TRUE(bool(file.open(tmp.path)));
        ASSERT_FALSE(bool(model::Qwen3Config::from_file(file, c)));
    }
    {
        TempFile tmp;  // no decoder layers
        tmp.write(serialise(skeleton(0, 256, 256, 128, 512, 32)));
        model::SafetensorsFile file;
        ASSERT_TRUE(bool(file.open(tmp.path)));
        ASSERT_FALSE(bool(model::Qwen3Config::from_file(file, c)));
    }
    {
        TempFile tmp;  // a query projection that is not whole heads of 128
        tmp.write(serialise(skeleton(1, 256, 192, 128, 512, 32)));
        model::SafetensorsFile file;
        ASSERT_TRUE(bool(file.open(tmp.path)));
        ASSERT_FALSE(bool(model::Qwen3Config::from_file(file, c)));
    }
    ASSERT_EQ(c.layers, 0);  // a refused file leaves the caller's config alone
}

TEST_CPU(test_qwen3_decoder, bf16_tensor_loader_rounds_f16_and_f32) {
    const std::vector<float> values{0.0f, 1.0f, -2.5f, 1.00390625f /* tie: rounds to even */, 3.14159274f, 65504.0f, 1e-8f};
    std::vector<uint16_t> as_bf16, as_f16;
    for (float v : values) {
        as_bf16.push_back(kxo_f32_to_bf16(v));
        as_f16.push_back(kxo_f32_to_f16(v));
    }
    const int64_t n = static_cast<int64_t>(values.size());
    std::vector<Blob> blobs;
    blobs.push_back(blob("a.bf16", "BF16", {n}, as_bf16));
    blobs.push_back(blob("a.f16", "F16", {n}, as_f16));
    blobs.push_back(blob("a.f32", "F32", {n}, values));
    blobs.push_back(blob("a.i64", "I64", {n}, std::vector<int64_t>(values.size(), 1)));
    TempFile tmp;
    tmp.write(serialise(blobs));
    model::SafetensorsFile file;
    ASSERT_TRUE(bool(file.open(tmp.path)));
    const std::vector<int32_t> dims{static_cast<int32_t>(n)};
    const base::DeviceType cpu = base::DeviceType::DeviceCPU;
    tensor::Tensor t;
    ASSERT_TRUE(bool(model::load_bf16_tensor(file, "a.bf16", dims, cpu, t)));
    ASSERT_EQ(std::memcmp(t.ptr<uint16_t>(), as_bf16.data(), as_bf16.size() * 2), 0);
    ASSERT_TRUE(bool(model::load_bf16_tensor(file, "a.f32", dims, cpu, t)));
    ASSERT_EQ(std::memcmp(t.ptr<uint16_t>(), as_bf16.data(), as_bf16.size() * 2), 0);
    ASSERT_TRUE(bool(model::load_bf16_tensor(file, "a.f16", dims, cpu, t)));
    for (size_t i = 0; i < values.size(); i++) {
        // fp16 -> fp32 is exact, so the expected bits are the bf16 rounding of the fp16 value
        ASSERT_EQ(t.ptr<uint16_t>()[i], kxo_f32_to_bf16(kxo_f16_to_f32(as_f16[i])));
    }
    ASSERT_TRUE(t.data_type() == base::DataType::DataTypeBf16);
    ASSERT_FALSE(bool(model::load_bf16_tensor(file, "a.i64", dims, cpu, t)));       // not a float type
    ASSERT_FALSE(bool(model::load_bf16_tensor(file, "a.none", dims, cpu, t)));      // absent
    ASSERT_FALSE(bool(model::load_bf16_tensor(file, "a.bf16", {3, 2}, cpu, t)));    // other shape
}

TEST_GPU(test_qwen3_decoder, step_checks_its_arguments) {
    model::Qwen3Decoder decoder(tiny_config(), 16);
    int32_t next = -1;
    ASSERT_FALSE(bool(decoder.step(1, 0, &next)));  // no weights yet
    ASSERT_FALSE(bool(decoder.capture()));
    decoder.init_random(1);
    ASSERT_FALSE(bool(decoder.step(1, 0, nullptr)));
    ASSERT_FALSE(bool(decoder.step(-1, 0, &next)));
    ASSERT_FALSE(bool(decoder.step(1024, 0, &next)));  // vocabulary is 0 .. 1023
    ASSERT_FALSE(bool(decoder.step(1, -1, &next)));
    ASSERT_FALSE(bool(decoder.step(1, 16, &next)));    // the caches hold positions 0 .. 15
    ASSERT_TRUE(bool(decoder.step(1023, 15, &next)));
    ASSERT_TRUE(next >= 0 && next < 1024);
    ASSERT_EQ(decoder.launches_per_step(), 1 + 2 * 5 + 3);
}

TEST_GPU(test_qwen3_decoder, graph_replay_is_the_step_launch_by_launch) {
    const int32_t tokens[] = {5, 900, 33, 33, 0, 1023, 17, 256};
    model::Qwen3Decoder eager(tiny_config(), 300), replayed(tiny_config(), 300);
    eager.init_random(42);
    replayed.init_random(42);
    eager.fill_cache_random(290, 3);
    replayed.fill_cache_random(290, 3);
    ASSERT_TRUE(bool(replayed.capture()));
    ASSERT_TRUE(replayed.captured());
    ASSERT_FALSE(eager.captured());
    for (int i = 0; i < 8; i++) {
        int32_t a = -1, b = -2;
        ASSERT_TRUE(bool(eager.step(tokens[i], 290 + i, &a)));
        ASSERT_TRUE(bool(replayed.step(tokens[i], 290 + i, &b)));
        ASSERT_EQ(a, b);
        const std::vector<uint16_t> la = eager.logits(), lb = replayed.logits();
        ASSERT_EQ(la.size(), size_t(1024));
        ASSERT_EQ(std::memcmp(la.data(), lb.data(), la.size() * 2), 0);
        for (uint16_t bits : la) ASSERT_TRUE((bits & 0x7F80) != 0x7F80);  // finite
    }
}

TEST_GPU(test_qwen3_decoder, random_init_depends_on_the_seed_only) {
    model::Qwen3Decoder a(tiny_config(), 8), b(tiny_config(), 8), c(tiny_config(), 8);
    a.init_random(7);
    b.init_random(7);
    c.init_random(8);
    int32_t na = -1, nb = -1, nc = -1;
    ASSERT_TRUE(bool(a.step(100, 0, &na)));
    ASSERT_TRUE(bool(b.step(100, 0, &nb)));
    ASSERT_TRUE(bool(c.step(100, 0, &nc)));
    const std::vector<uint16_t> la = a.logits(), lb = b.logits(), lc = c.logits();
    ASSERT_EQ(na, nb);
    ASSERT_EQ(std::memcmp(la.data(), lb.data(), la.size() * 2), 0);
    ASSERT_TRUE(std::memcmp(la.data(), lc.data(), la.size() * 2) != 0);
    double ms = 0.0;
    ASSERT_FALSE(bool(a.time_steps(100, 1, 0, 0, &ms)));  // at least one timed step
    ASSERT_TRUE(bool(a.time_steps(100, 1, 3, 1, &ms)));
    ASSERT_TRUE(ms > 0.0);
}

TEST_GPU(test_qwen3_decoder, fused_layers_return_the_bits_of_the_fused_entry_points) {
    // The five launches of a decoder layer as forward() calls of kuiper layers (MatmulLayer::set_fusion,
    // MultiHeadAttention::forward_chunks) against the same launches made through the C ABI directly: the same
    // kernels on the same operands, except that the first layer's row is normed by a launch of its own, which
    // returns the bits of the norm inside the launch.
    model::Qwen3Decoder fused(tiny_config(), 64), layers(tiny_config(), 64, model::DecodePath::Layers);
    fused.init_random(11);
    layers.init_random(11);
    ASSERT_TRUE(layers.path() == model::DecodePath::Layers);
    ASSERT_EQ(layers.launches_per_step(), fused.launches_per_step() + 1);
    const int32_t tokens[] = {9, 400, 77, 1000, 3, 3};
    for (int i = 0; i < 6; i++) {
        int32_t a = -1, b = -2;
        ASSERT_TRUE(bool(fused.step(tokens[i], i, &a)));
        ASSERT_TRUE(bool(layers.step(tokens[i], i, &b)));
        ASSERT_EQ(a, b);
        const std::vector<uint16_t> la = fused.logits(), lb = layers.logits();
        ASSERT_EQ(std::memcmp(la.data(), lb.data(), la.size() * 2), 0);
    }
    // and from a captured graph
    model::Qwen3Decoder replayed(tiny_config(), 64, model::DecodePath::Layers);
    replayed.init_random(11);
    ASSERT_TRUE(bool(replayed.capture()));
    for (int i = 0; i < 6; i++) {
        int32_t a = -1, b = -2;
        ASSERT_TRUE(bool(fused.step(tokens[i], i, &a)));
        ASSERT_TRUE(bool(replayed.step(tokens[i], i, &b)));
        ASSERT_EQ(a, b);
        const std::vector<uint16_t> la = fused.logits(), lb = replayed.logits();
        ASSERT_EQ(std::memcmp(la.data(), lb.data(), la.size() * 2), 0);
    }
}

TEST_GPU(test_qwen3_decoder, a_fused_form_is_refused_where_it_does_not_exist) {
    op::MatmulLayer host(base::DeviceType::DeviceCPU, 256, 256, true, 128);
    op::MatmulLayer dense(base::DeviceType::DeviceCUDA, 256, 256, false);
    kernel::MatmulChain chain;
    ASSERT_FALSE(bool(host.set_fusion(chain)));
    ASSERT_FALSE(bool(dense.set_fusion(chain)));
    ASSERT_FALSE(host.fused());
}

TEST_GPU(test_qwen3_decoder, operator_by_operator_path_agrees_with_the_fused_path) {
    // Same weights, same tokens: one forward() per operator against the fused entry points.  The fused
    // path adds up the sum of squares of the RMSNorm tile by tile, so the logits agree to rounding.
    model::Qwen3Decoder fused(tiny_config(), 64), layers(tiny_config(), 64, model::DecodePath::Operators);
    fused.init_random(11);
    layers.init_random(11);
    ASSERT_TRUE(layers.path() == model::DecodePath::Operators);
    ASSERT_EQ(layers.launches_per_step(), 1 + 2 * 10 + 3);
    const int32_t tokens[] = {9, 400, 77, 1000, 3, 3};
    for (int i = 0; i < 6; i++) {
        int32_t a = -1, b = -1;
        ASSERT_TRUE(bool(fused.step(tokens[i], i, &a)));
        ASSERT_TRUE(bool(layers.step(tokens[i], i, &b)));
        const std::vector<uint16_t> la = fused.logits(), lb = layers.logits();
        double num = 0.0, den = 0.0;
        for (size_t k = 0; k < la.size(); k++) {
            const double x = kxo_bf16_to_f32(la[k]), y = kxo_bf16_to_f32(lb[k]);
            num += (x - y) * (x - y);
            den += y * y;
        }
        ASSERT_TRUE(den > 0.0);
        ASSERT_LE(std::sqrt(num / den), 2e-2);
    }
}

TEST_GPU(test_qwen3_decoder, operator_by_operator_path_can_be_captured) {
    model::Qwen3Decoder eager(tiny_config(), 40, model::DecodePath::Operators);
    model::Qwen3Decoder replayed(tiny_config(), 40, model::DecodePath::Operators);
    eager.init_random(5);
    replayed.init_random(5);
    ASSERT_TRUE(bool(replayed.capture()));  // nothing may allocate while the stream is captured
    for (int i = 0; i < 5; i++) {
        int32_t a = -1, b = -2;
        ASSERT_TRUE(bool(eager.step(100 + i, i, &a)));
        ASSERT_TRUE(bool(replayed.step(100 + i, i, &b)));
        ASSERT_EQ(a, b);
        const std::vector<uint16_t> la = eager.logits(), lb = replayed.logits();
        ASSERT_EQ(std::memcmp(la.data(), lb.data(), la.size() * 2), 0);
    }
}
