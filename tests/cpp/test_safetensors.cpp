// The checkpoint reader (model/safetensors.h): files written here byte by byte to the format's
// definition, read back through SafetensorsFile, attached to MatmulLayer objects and run against
// the CPU oracle (oracle/kx_oracle.c, the checker linked into this binary).
#include <hip/hip_runtime_api.h>
#include <unistd.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../oracle/kx_oracle.h"
#include "mini_test.h"
#include "model/safetensors.h"
#include "safetensors_writer.h"
#include "op/matmul.h"

namespace {

using namespace stw;

struct AwqTensors {
    int K, N, G;
    std::vector<int32_t> qweight, qzeros;
    std::vector<uint16_t> scales;
};

AwqTensors make_awq(int K, int N, int G, uint64_t seed) {
    AwqTensors t{K, N, G, {}, {}, {}};
    Rng rng(seed);
    t.qweight.resize(size_t(K) * N / 8);
    for (auto& v : t.qweight) v = int32_t(rng.next());
    t.qzeros.resize(size_t(K / G) * N / 8);
    for (auto& v : t.qzeros) v = int32_t(rng.next());
    t.scales.resize(size_t(K / G) * N);
    for (auto& v : t.scales) v = kxo_f32_to_f16(float(0.001 + 0.019 * rng.uniform()));
    return t;
}

void add_awq(std::vector<Blob>& blobs, const std::string& prefix, const AwqTensors& t) {
    // scales first, then zeros, then weights: the reader must not depend on the order
    blobs.push_back(blob(prefix + ".scales", "F16", {t.K / t.G, t.N}, t.scales));
    blobs.push_back(blob(prefix + ".qzeros", "I32", {t.K / t.G, t.N / 8}, t.qzeros));
    blobs.push_back(blob(prefix + ".qweight", "I32", {t.K, t.N / 8}, t.qweight));
}

std::vector<uint16_t> random_bf16(size_t n, uint64_t seed) {
    Rng rng(seed);
    std::vector<uint16_t> v(n);
    for (auto& e : v) e = kxo_f32_to_bf16(float(rng.normal()));
    return v;
}

// runs `layer` (weights already attached) on x [M, K] and returns y [M, N] as bf16 bits
std::vector<uint16_t> run_layer(op::MatmulLayer& layer, std::vector<uint16_t>& x, int M) {
    const bool gpu = layer.device_type() == base::DeviceType::DeviceCUDA;
    const int K = layer.dim1(), N = layer.dim0();
    std::vector<uint16_t> out(size_t(M) * N, 0x7FC0);
    tensor::Tensor tx(base::DataType::DataTypeBf16, {M, K}, false, nullptr, x.data());
    tensor::Tensor ty(base::DataType::DataTypeBf16, {M, N}, false, nullptr, out.data());
    tx.set_device_type(base::DeviceType::DeviceCPU);
    ty.set_device_type(base::DeviceType::DeviceCPU);
    if (gpu) {
        tx.to_cuda();
        ty.to_cuda();
        if (layer.cuda_config() == nullptr) {
            auto config = std::make_shared<kernel::CudaConfig>();
            config->create();
            layer.set_cuda_config(config);
        }
    }
    const base::Status st = layer.forward(tx, ty);
    ASSERT_TRUE(bool(st));
    if (gpu) {
        ASSERT_EQ(hipDeviceSynchronize(), hipSuccess);
        ty.to_cpu();
        std::memcpy(out.data(), ty.ptr<uint16_t>(), out.size() * 2);
    }
    return out;
}

void expect_close(const std::vector<uint16_t>& got, const std::vector<double>& ref) {
    double num = 0, den = 0;
    for (size_t i = 0; i < ref.size(); i++) {
        const double r = kxo_bf16_to_f32(kxo_f32_to_bf16(float(ref[i])));
        const double g = kxo_bf16_to_f32(got[i]);
        ASSERT_TRUE(std::isfinite(g));
        num += (g - r) * (g - r);
        den += r * r;
    }
    ASSERT_LE(std::sqrt(num / den), 1e-3);
}

void loaded_layer_matches_oracle(base::DeviceType device) {
    const int M = 2, K = 512, N = 1024, G = 128;
    AwqTensors t = make_awq(K, N, G, 11);
    std::vector<Blob> blobs;
    blobs.push_back(blob("unrelated.bias", "F32", {3}, std::vector<float>{1.f, 2.f, 3.f}));
    add_awq(blobs, "model.layers.0.self_attn.o_proj", t);
    TempFile tmp;
    tmp.write(serialise(blobs));

    op::MatmulLayer layer(device, N, K, true, G);
    {
        model::SafetensorsFile file;
        ASSERT_TRUE(bool(file.open(tmp.path)));
        ASSERT_TRUE(bool(model::load_awq_linear(file, "model.layers.0.self_attn.o_proj", layer)));
    }  // the file is closed: the layer owns copies
    std::vector<uint16_t> x = random_bf16(size_t(M) * K, 5);
    std::vector<uint16_t> y = run_layer(layer, x, M);
    std::vector<double> ref(size_t(M) * N);
    ASSERT_EQ(kxo_gemv_awq_f64(x.data(), t.qweight.data(), t.scales.data(), t.qzeros.data(), M, K, N, G, ref.data()), 0);
    expect_close(y, ref);
}

void fused_load_equals_separate_layers(base::DeviceType device) {
    const int K = 512, G = 128;
    const int ns[3] = {512, 128, 128};  // q | k | v
    const char* names[3] = {"attn.q_proj", "attn.k_proj", "attn.v_proj"};
    std::vector<Blob> blobs;
    std::vector<AwqTensors> parts;
    for (int i = 0; i < 3; i++) {
        parts.push_back(make_awq(K, ns[i], G, 100 + i));
        add_awq(blobs, names[i], parts.back());
    }
    TempFile tmp;
    tmp.write(serialise(blobs));
    model::SafetensorsFile file;
    ASSERT_TRUE(bool(file.open(tmp.path)));

    std::vector<uint16_t> x = random_bf16(K, 9);
    op::MatmulLayer fused(device, ns[0] + ns[1] + ns[2], K, true, G);
    ASSERT_TRUE(bool(model::load_awq_linear_fused(file, {names[0], names[1], names[2]}, fused)));
    std::vector<uint16_t> y_fused = run_layer(fused, x, 1);
    size_t at = 0;
    for (int i = 0; i < 3; i++) {
        op::MatmulLayer single(device, ns[i], K, true, G);
        ASSERT_TRUE(bool(model::load_awq_linear(file, names[i], single)));
        std::vector<uint16_t> y = run_layer(single, x, 1);
        for (int n = 0; n < ns[i]; n++) ASSERT_EQ(y_fused[at + n], y[n]);  // same K split, same order: same bits
        at += ns[i];
    }
    // a fused layer whose width does not match the parts is refused
    op::MatmulLayer wrong(device, ns[0] + ns[1], K, true, G);
    ASSERT_FALSE(bool(model::load_awq_linear_fused(file, {names[0], names[1], names[2]}, wrong)));
}

}  // namespace

TEST_CPU(test_safetensors, header_and_data_round_trip) {
    std::vector<int32_t> a{1, -2, 3, -4, 5, -6};
    std::vector<uint16_t> b{0x3F80, 0xBF80, 0x7FC0};
    std::vector<Blob> blobs{blob("a.b.c", "I32", {2, 3}, a), blob("weird \\\"name\\\" \\u00e9", "BF16", {3}, b),
                            blob("empty", "F16", {0, 4}, std::vector<uint16_t>{})};
    TempFile tmp;
    tmp.write(serialise(blobs, "{\"format\":\"pt\",\"note\":\"x\\ny\"}"));
    model::SafetensorsFile file;
    ASSERT_TRUE(bool(file.open(tmp.path)));
    ASSERT_EQ(file.entries().size(), size_t(3));
    const model::TensorEntry* e = file.find("a.b.c");
    ASSERT_TRUE(e != nullptr);
    ASSERT_EQ(e->dtype, std::string("I32"));
    ASSERT_EQ(e->shape.size(), size_t(2));
    ASSERT_EQ(e->shape[0], 2);
    ASSERT_EQ(e->shape[1], 3);
    ASSERT_EQ(std::memcmp(file.data(*e), a.data(), 24), 0);
    const model::TensorEntry* w = file.find("weird \"name\" \xC3\xA9");  // escapes decoded, UTF-8
    ASSERT_TRUE(w != nullptr);
    ASSERT_EQ(std::memcmp(file.data(*w), b.data(), 6), 0);
    ASSERT_EQ(file.find("empty")->byte_size(), size_t(0));
    ASSERT_TRUE(file.find("missing") == nullptr);
    ASSERT_EQ(file.metadata().at("format"), std::string("pt"));
    ASSERT_EQ(file.metadata().at("note"), std::string("x\ny"));
    file.close();
    ASSERT_FALSE(file.is_open());
}

TEST_CPU(test_safetensors, malformed_files_are_refused) {
    TempFile tmp;
    model::SafetensorsFile file;
    ASSERT_FALSE(bool(file.open("/nonexistent/dir/x.safetensors")));
    tmp.write("short");
    ASSERT_FALSE(bool(file.open(tmp.path)));
    tmp.write(with_length_prefix("{}", "").substr(0, 8) + "{");  // header length says 2, file holds 1
    ASSERT_FALSE(bool(file.open(tmp.path)));
    const char* bad_headers[] = {
        "[1,2]",                                                              // not an object
        "{\"t\":{\"dtype\":\"I32\",\"shape\":[2],\"data_offsets\":[0,4]}}",    // 4 bytes for 2 x I32
        "{\"t\":{\"dtype\":\"I32\",\"shape\":[2],\"data_offsets\":[0,16]}}",   // beyond the 8 data bytes
        "{\"t\":{\"dtype\":\"I32\",\"shape\":[2],\"data_offsets\":[8,0]}}",    // end before begin
        "{\"t\":{\"dtype\":\"Q4\",\"shape\":[8],\"data_offsets\":[0,8]}}",     // unknown dtype
        "{\"t\":{\"dtype\":\"I32\",\"shape\":[-2],\"data_offsets\":[0,8]}}",   // negative extent
        "{\"t\":{\"dtype\":\"I32\",\"shape\":[2]}}",                           // no offsets
        "{\"t\":{\"dtype\":\"I32\",\"shape\":[2],\"data_offsets\":[0,8]},"
        "\"t\":{\"dtype\":\"I32\",\"shape\":[2],\"data_offsets\":[0,8]}}",     // twice
        "{\"t\":{\"dtype\":\"I32\",\"shape\":[2],\"data_offsets\":[0,8]}",     // unterminated
        "{\"t\":{\"dtype\":\"I32\",\"shape\":[2],\"data_offsets\":[0,8]}} x",  // trailing garbage
    };
    for (const char* h : bad_headers) {
        tmp.write(with_length_prefix(h, std::string(8, '\1')));
        ASSERT_FALSE(bool(file.open(tmp.path)));
        ASSERT_FALSE(file.is_open());
    }
    // the well-formed neighbour of the cases above is accepted
    tmp.write(with_length_prefix("{\"t\":{\"dtype\":\"I32\",\"shape\":[2],\"data_offsets\":[0,8]}}", std::string(8, '\1')));
    ASSERT_TRUE(bool(file.open(tmp.path)));
}

TEST_CPU(test_safetensors, awq_shapes_are_checked_against_the_layer) {
    AwqTensors t = make_awq(256, 64, 128, 3);
    std::vector<Blob> blobs;
    add_awq(blobs, "p", t);
    blobs.push_back(blob("q.qweight", "I32", {256, 8}, t.qweight));  // q has no zeros and scales
    blobs.push_back(blob("w", "BF16", {4, 8}, std::vector<uint16_t>(32, 0x3F80)));
    TempFile tmp;
    tmp.write(serialise(blobs));
    model::SafetensorsFile file;
    ASSERT_TRUE(bool(file.open(tmp.path)));
    op::MatmulLayer ok(base::DeviceType::DeviceCPU, 64, 256, true, 128);
    ASSERT_TRUE(bool(model::load_awq_linear(file, "p", ok)));
    op::MatmulLayer wrong_n(base::DeviceType::DeviceCPU, 128, 256, true, 128);
    ASSERT_FALSE(bool(model::load_awq_linear(file, "p", wrong_n)));
    op::MatmulLayer wrong_k(base::DeviceType::DeviceCPU, 64, 512, true, 128);
    ASSERT_FALSE(bool(model::load_awq_linear(file, "p", wrong_k)));
    op::MatmulLayer wrong_group(base::DeviceType::DeviceCPU, 64, 256, true, 64);
    ASSERT_FALSE(bool(model::load_awq_linear(file, "p", wrong_group)));
    ASSERT_FALSE(bool(model::load_awq_linear(file, "q", ok)));
    ASSERT_FALSE(bool(model::load_awq_linear(file, "absent", ok)));
    op::MatmulLayer plain(base::DeviceType::DeviceCPU, 4, 8, false);
    ASSERT_FALSE(bool(model::load_awq_linear(file, "p", plain)));
    ASSERT_TRUE(bool(model::load_bf16_linear(file, "w", plain)));
    op::MatmulLayer plain_wrong(base::DeviceType::DeviceCPU, 8, 4, false);
    ASSERT_FALSE(bool(model::load_bf16_linear(file, "w", plain_wrong)));
    ASSERT_FALSE(bool(model::load_bf16_linear(file, "w", ok)));
}

TEST_CPU(test_safetensors, loaded_layer_matches_oracle_cpu) { loaded_layer_matches_oracle(base::DeviceType::DeviceCPU); }
TEST_GPU(test_safetensors, loaded_layer_matches_oracle_cuda) { loaded_layer_matches_oracle(base::DeviceType::DeviceCUDA); }
TEST_CPU(test_safetensors, fused_load_equals_separate_layers_cpu) {
    fused_load_equals_separate_layers(base::DeviceType::DeviceCPU);
}
TEST_GPU(test_safetensors, fused_load_equals_separate_layers_cuda) {
    fused_load_equals_separate_layers(base::DeviceType::DeviceCUDA);
}
