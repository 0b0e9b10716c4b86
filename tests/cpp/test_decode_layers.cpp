// The decode-step operator layers (RmsNormLayer, SwiGLULayer, EmbeddingLayer, RoPELayer,
// MultiHeadAttention): the host kernels against closed forms on small cases, and the GPU layers
// against the host layers on random inputs.  bf16 helpers come from the CPU oracle linked into this
// binary (oracle/kx_oracle.c), which is pinned exhaustively against library casts.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstring>
#include <vector>

#include "../../oracle/kx_oracle.h"
#include "mini_test.h"
#include "op/embedding.h"
#include "op/mha.h"
#include "op/rmsnorm.h"
#include "op/rope.h"
#include "op/swiglu.h"

namespace {

using base::DataType;
using base::DeviceType;

struct Rng {  // SplitMix64
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed) {}
    uint64_t next() {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double uniform() { return double(next() >> 11) * (1.0 / 9007199254740992.0); }
    double normal() { return std::sqrt(-2.0 * std::log(1.0 - uniform())) * std::cos(6.283185307179586 * uniform()); }
};

uint16_t bf(float v) { return kxo_f32_to_bf16(v); }
float fl(uint16_t h) { return kxo_bf16_to_f32(h); }

std::vector<uint16_t> random_bf16(size_t n, uint64_t seed, double scale = 1.0, double shift = 0.0) {
    Rng rng(seed);
    std::vector<uint16_t> v(n);
    for (auto& e : v) e = bf(float(shift + scale * rng.normal()));
    return v;
}

// A tensor over caller memory on the host, or a copy of it on the GPU.
template <typename T>
tensor::Tensor make(DataType type, std::vector<int32_t> dims, std::vector<T>& data, DeviceType device) {
    tensor::Tensor t(type, std::move(dims), false, nullptr, data.data());
    t.set_device_type(DeviceType::DeviceCPU);
    if (device == DeviceType::DeviceCUDA) t.to_cuda();
    return t;
}

template <typename T>
std::vector<T> fetch(tensor::Tensor t) {
    if (t.device_type() == DeviceType::DeviceCUDA) {
        ASSERT_EQ(hipDeviceSynchronize(), hipSuccess);
        t.to_cpu();
    }
    std::vector<T> out(t.size());
    std::memcpy(out.data(), t.ptr<T>(), out.size() * sizeof(T));
    return out;
}

// |a - b| <= ulps bf16 units in the last place of max(|a|, |b|), element by element
void expect_ulps(const std::vector<uint16_t>& a, const std::vector<uint16_t>& b, double ulps) {
    ASSERT_EQ(a.size(), b.size());
    for (size_t i = 0; i < a.size(); i++) {
        const double x = fl(a[i]), y = fl(b[i]);
        ASSERT_TRUE(std::isfinite(x) && std::isfinite(y));
        const double mag = std::fmax(std::fabs(x), std::fabs(y));
        const double unit = mag > 0 ? std::pow(2.0, std::floor(std::log2(mag)) - 7) : 0.0;
        if (std::fabs(x - y) > ulps * unit + 1e-30) {
            KX_FAIL("element " + std::to_string(i) + ": " + std::to_string(x) + " vs " + std::to_string(y));
        }
    }
}

// ------------------------------------------------------------------ runners (host or GPU)
std::vector<uint16_t> run_rmsnorm(DeviceType dev, int rows, int dim, std::vector<uint16_t> x, std::vector<uint16_t> delta,
                                  std::vector<uint16_t> gain, float eps, std::vector<uint16_t>* x_after = nullptr) {
    op::RmsNormLayer layer(dev, dim, eps);
    std::vector<uint16_t> y(x.size(), 0x7FC0);
    tensor::Tensor tx = make(DataType::DataTypeBf16, {rows, dim}, x, dev);
    tensor::Tensor ty = make(DataType::DataTypeBf16, {rows, dim}, y, dev);
    tensor::Tensor tg = make(DataType::DataTypeBf16, {dim}, gain, dev);
    ASSERT_TRUE(bool(layer.set_weight(0, tg)));
    base::Status st;
    if (delta.empty()) {
        st = layer.forward(tx, ty);
    } else {
        tensor::Tensor td = make(DataType::DataTypeBf16, {rows, dim}, delta, dev);
        st = layer.forward(tx, td, ty);
    }
    ASSERT_TRUE(bool(st));
    if (x_after) *x_after = fetch<uint16_t>(tx);
    return fetch<uint16_t>(ty);
}

std::vector<uint16_t> run_swiglu(DeviceType dev, std::vector<uint16_t> gate, std::vector<uint16_t> up) {
    const int n = int(gate.size());
    op::SwiGLULayer layer(dev, n);
    std::vector<uint16_t> y(n, 0x7FC0);
    tensor::Tensor tg = make(DataType::DataTypeBf16, {n}, gate, dev);
    tensor::Tensor tu = make(DataType::DataTypeBf16, {n}, up, dev);
    tensor::Tensor ty = make(DataType::DataTypeBf16, {n}, y, dev);
    ASSERT_TRUE(bool(layer.forward(tg, tu, ty)));
    return fetch<uint16_t>(ty);
}

std::vector<uint16_t> run_embedding(DeviceType dev, int vocab, int dim, std::vector<uint16_t> table, int32_t token) {
    op::EmbeddingLayer layer(dev, vocab, dim);
    std::vector<int32_t> tok{token};
    std::vector<uint16_t> y(dim, 0x7FC0);
    tensor::Tensor tt = make(DataType::DataTypeBf16, {vocab, dim}, table, dev);
    tensor::Tensor ti = make(DataType::DataTypeInt32, {1}, tok, dev);
    tensor::Tensor ty = make(DataType::DataTypeBf16, {dim}, y, dev);
    ASSERT_TRUE(bool(layer.set_weight(0, tt)));
    ASSERT_TRUE(bool(layer.forward(ti, ty)));
    return fetch<uint16_t>(ty);
}

struct RopeResult {
    std::vector<uint16_t> q, k_cache, v_cache;
};

RopeResult run_rope(DeviceType dev, int n_q, int n_kv, int max_pos, int32_t pos, std::vector<uint16_t> qkv,
                    std::vector<uint16_t> q_gain, std::vector<uint16_t> k_gain, float theta, float eps) {
    op::RoPELayer layer(dev, n_q, n_kv, theta, eps);
    std::vector<int32_t> p{pos};
    std::vector<uint16_t> q(size_t(n_q) * 128, 0x7FC0), kc(size_t(max_pos) * n_kv * 128, bf(3.0f)), vc(kc.size(), bf(5.0f));
    tensor::Tensor tqkv = make(DataType::DataTypeBf16, {(n_q + 2 * n_kv) * 128}, qkv, dev);
    tensor::Tensor tp = make(DataType::DataTypeInt32, {1}, p, dev);
    tensor::Tensor tk = make(DataType::DataTypeBf16, {max_pos, n_kv, 128}, kc, dev);
    tensor::Tensor tv = make(DataType::DataTypeBf16, {max_pos, n_kv, 128}, vc, dev);
    tensor::Tensor tq = make(DataType::DataTypeBf16, {n_q * 128}, q, dev);
    tensor::Tensor tqg = make(DataType::DataTypeBf16, {128}, q_gain, dev);
    tensor::Tensor tkg = make(DataType::DataTypeBf16, {128}, k_gain, dev);
    ASSERT_TRUE(bool(layer.set_weight(0, tqg)));
    ASSERT_TRUE(bool(layer.set_weight(1, tkg)));
    ASSERT_TRUE(bool(layer.forward(tqkv, tp, tk, tv, tq)));
    return {fetch<uint16_t>(tq), fetch<uint16_t>(tk), fetch<uint16_t>(tv)};
}

std::vector<uint16_t> run_mha(DeviceType dev, int n_q, int n_kv, int max_pos, int32_t pos, std::vector<uint16_t> q,
                              std::vector<uint16_t> kc, std::vector<uint16_t> vc) {
    op::MultiHeadAttention layer(dev, n_q, n_kv);
    std::vector<int32_t> p{pos};
    std::vector<uint16_t> out(q.size(), 0x7FC0);
    tensor::Tensor tq = make(DataType::DataTypeBf16, {n_q * 128}, q, dev);
    tensor::Tensor tp = make(DataType::DataTypeInt32, {1}, p, dev);
    tensor::Tensor tk = make(DataType::DataTypeBf16, {max_pos, n_kv, 128}, kc, dev);
    tensor::Tensor tv = make(DataType::DataTypeBf16, {max_pos, n_kv, 128}, vc, dev);
    tensor::Tensor to = make(DataType::DataTypeBf16, {n_q * 128}, out, dev);
    ASSERT_TRUE(bool(layer.forward(tq, tp, tk, tv, to)));
    return fetch<uint16_t>(to);
}

}  // namespace

// ------------------------------------------------------------------ host kernels against closed forms
TEST_CPU(test_decode_layers, rmsnorm_closed_form) {
    const float eps = 1e-6f;
    std::vector<uint16_t> x(8, 0), gain(8, bf(1.0f));
    x[0] = bf(3.0f);
    x[1] = bf(4.0f);
    gain[1] = bf(0.5f);
    std::vector<uint16_t> y = run_rmsnorm(DeviceType::DeviceCPU, 1, 8, x, {}, gain, eps);
    const double inv = 1.0 / std::sqrt(25.0 / 8.0 + eps);
    ASSERT_EQ(y[0], bf(float(3.0 * inv)));
    ASSERT_EQ(y[1], bf(0.5f * fl(bf(float(4.0 * inv)))));
    for (int i = 2; i < 8; i++) ASSERT_EQ(fl(y[i]), 0.0f);
    // with a delta the input row becomes bf16(x + delta) and the norm is taken of that
    std::vector<uint16_t> delta(8, 0), after;
    delta[0] = bf(-3.0f);
    delta[2] = bf(3.0f);  // row becomes (0, 4, 3, 0...): same mean square
    y = run_rmsnorm(DeviceType::DeviceCPU, 1, 8, x, delta, gain, eps, &after);
    ASSERT_EQ(fl(after[0]), 0.0f);
    ASSERT_EQ(fl(after[2]), 3.0f);
    ASSERT_EQ(y[2], bf(float(3.0 * inv)));
    ASSERT_EQ(fl(y[0]), 0.0f);
}

TEST_CPU(test_decode_layers, swiglu_closed_form) {
    std::vector<uint16_t> gate{bf(0.0f), bf(1.0f), bf(-1.0f), bf(8.0f)}, up{bf(7.0f), bf(2.0f), bf(2.0f), bf(-0.5f)};
    std::vector<uint16_t> y = run_swiglu(DeviceType::DeviceCPU, gate, up);
    ASSERT_EQ(fl(y[0]), 0.0f);
    ASSERT_EQ(y[1], bf(fl(bf(float(1.0 / (1.0 + std::exp(-1.0))))) * 2.0f));
    ASSERT_EQ(y[2], bf(fl(bf(float(-1.0 / (1.0 + std::exp(1.0))))) * 2.0f));
    ASSERT_EQ(y[3], bf(fl(bf(float(8.0 / (1.0 + std::exp(-8.0))))) * -0.5f));
}

TEST_CPU(test_decode_layers, embedding_copies_and_clamps) {
    std::vector<uint16_t> table = random_bf16(5 * 16, 1);
    for (int32_t token : {0, 3, 4}) {
        std::vector<uint16_t> y = run_embedding(DeviceType::DeviceCPU, 5, 16, table, token);
        for (int i = 0; i < 16; i++) ASSERT_EQ(y[i], table[size_t(token) * 16 + i]);
    }
    std::vector<uint16_t> low = run_embedding(DeviceType::DeviceCPU, 5, 16, table, -7);
    std::vector<uint16_t> high = run_embedding(DeviceType::DeviceCPU, 5, 16, table, 99);
    for (int i = 0; i < 16; i++) {
        ASSERT_EQ(low[i], table[i]);
        ASSERT_EQ(high[i], table[4 * 16 + i]);
    }
}

TEST_CPU(test_decode_layers, rope_closed_form) {
    const int n_q = 1, n_kv = 1, max_pos = 4;
    const float eps = 1e-6f, theta = 1e6f;
    std::vector<uint16_t> qkv(3 * 128, 0), gain(128, bf(1.0f));
    qkv[0] = bf(2.0f);                   // q: one non-zero element, partner 64 is zero
    qkv[128 + 5] = bf(-3.0f);            // k: element 5
    for (int i = 0; i < 128; i++) qkv[256 + i] = bf(float(i) * 0.25f);  // v: copied as is
    // position 0: no rotation; the head is sqrt(128) * sign in the non-zero slot
    RopeResult r0 = run_rope(DeviceType::DeviceCPU, n_q, n_kv, max_pos, 0, qkv, gain, gain, theta, eps);
    const float n0 = fl(bf(float(2.0 / std::sqrt(4.0 / 128.0 + eps))));
    ASSERT_EQ(r0.q[0], bf(n0));
    for (int i = 1; i < 128; i++) ASSERT_EQ(fl(r0.q[i]), 0.0f);
    // position 1: element 0 has frequency 1, so (n, 0) turns into (n cos 1, n sin 1)
    RopeResult r1 = run_rope(DeviceType::DeviceCPU, n_q, n_kv, max_pos, 1, qkv, gain, gain, theta, eps);
    expect_ulps({r1.q[0], r1.q[64]}, {bf(n0 * float(std::cos(1.0))), bf(n0 * float(std::sin(1.0)))}, 1.0);
    // key: element 5 has frequency theta^(-5/64); it lands in row 1 of the cache, other rows untouched
    const double f5 = std::pow(double(theta), -5.0 / 64.0);
    const float nk = fl(bf(float(-3.0 / std::sqrt(9.0 / 128.0 + eps))));
    expect_ulps({r1.k_cache[128 + 5], r1.k_cache[128 + 69]},
                {bf(nk * float(std::cos(f5))), bf(nk * float(std::sin(f5)))}, 1.0);
    ASSERT_EQ(r1.k_cache[0], bf(3.0f));
    ASSERT_EQ(r1.k_cache[2 * 128], bf(3.0f));
    for (int i = 0; i < 128; i++) ASSERT_EQ(r1.v_cache[128 + i], qkv[256 + i]);
    ASSERT_EQ(r1.v_cache[0], bf(5.0f));
}

TEST_CPU(test_decode_layers, mha_closed_form) {
    const int n_q = 2, n_kv = 1, max_pos = 4;
    std::vector<uint16_t> kc(size_t(max_pos) * 128, 0), vc(kc.size(), 0), q(2 * 128, 0);
    for (int t = 0; t < max_pos; t++) {
        for (int i = 0; i < 128; i++) vc[size_t(t) * 128 + i] = bf(float(t + 1) + float(i) * 0.125f);
    }
    // one cached position: the output is that value row, whatever the query
    q[3] = bf(1.5f);
    std::vector<uint16_t> y = run_mha(DeviceType::DeviceCPU, n_q, n_kv, max_pos, 0, q, kc, vc);
    for (int i = 0; i < 128; i++) ASSERT_EQ(y[i], vc[i]);
    // zero keys: uniform weights over positions 0..2, the mean of three rows (head 1 likewise)
    y = run_mha(DeviceType::DeviceCPU, n_q, n_kv, max_pos, 2, q, kc, vc);
    for (int i = 0; i < 128; i++) {
        const float mean = (fl(vc[i]) + fl(vc[128 + i]) + fl(vc[256 + i])) / 3.0f;
        expect_ulps({y[i], y[128 + i]}, {bf(mean), bf(mean)}, 1.0);
    }
    // a key aligned with head 0's query and a large score: that position takes all the weight
    kc[1 * 128 + 3] = bf(200.0f);  // score 1.5 * 200 / sqrt(128) = 26.5 against 0
    y = run_mha(DeviceType::DeviceCPU, n_q, n_kv, max_pos, 2, q, kc, vc);
    for (int i = 0; i < 128; i++) ASSERT_EQ(y[i], vc[128 + i]);
    for (int i = 0; i < 128; i++) {  // head 1 (zero query) still averages
        const float mean = (fl(vc[i]) + fl(vc[128 + i]) + fl(vc[256 + i])) / 3.0f;
        expect_ulps({y[128 + i]}, {bf(mean)}, 1.0);
    }
}

TEST_CPU(test_decode_layers, shape_errors_are_reported) {
    std::vector<uint16_t> a(16, bf(1.0f)), b(8, bf(1.0f));
    op::SwiGLULayer swiglu(DeviceType::DeviceCPU, 16);
    tensor::Tensor ta = make(DataType::DataTypeBf16, {16}, a, DeviceType::DeviceCPU);
    tensor::Tensor tb = make(DataType::DataTypeBf16, {8}, b, DeviceType::DeviceCPU);
    ASSERT_FALSE(bool(swiglu.forward(ta, tb, ta)));
    op::RmsNormLayer norm(DeviceType::DeviceCPU, 16);
    ASSERT_FALSE(bool(norm.forward(ta, ta)));  // no gain attached
    ASSERT_TRUE(bool(norm.set_weight(0, ta)));
    ASSERT_TRUE(bool(norm.forward(ta, ta)));
    ASSERT_FALSE(bool(norm.forward(tb, tb)));  // rows of 8 in a layer of 16
    op::MultiHeadAttention mha(DeviceType::DeviceCPU, 3, 2);
    ASSERT_FALSE(bool(mha.forward()));
}

// ------------------------------------------------------------------ GPU layers against the host layers
TEST_GPU(test_decode_layers, rmsnorm_cuda_matches_cpu) {
    for (int dim : {4096, 5120, 264}) {
        const int rows = 3;
        std::vector<uint16_t> x = random_bf16(size_t(rows) * dim, 11, 2.0), d = random_bf16(size_t(rows) * dim, 12);
        std::vector<uint16_t> g = random_bf16(dim, 13, 0.1, 1.0), after_cpu, after_gpu;
        // the two sides add the squares in different orders: the normalised value may round the other way,
        // and the product with the gain is rounded once more
        expect_ulps(run_rmsnorm(DeviceType::DeviceCUDA, rows, dim, x, {}, g, 1e-6f),
                    run_rmsnorm(DeviceType::DeviceCPU, rows, dim, x, {}, g, 1e-6f), 2.0);
        expect_ulps(run_rmsnorm(DeviceType::DeviceCUDA, rows, dim, x, d, g, 1e-6f, &after_gpu),
                    run_rmsnorm(DeviceType::DeviceCPU, rows, dim, x, d, g, 1e-6f, &after_cpu), 2.0);
        ASSERT_TRUE(after_cpu == after_gpu);  // the residual add is one rounding: same bits
    }
}

TEST_GPU(test_decode_layers, swiglu_and_embedding_cuda_match_cpu) {
    std::vector<uint16_t> gate = random_bf16(12288, 21, 2.0), up = random_bf16(12288, 22);
    expect_ulps(run_swiglu(DeviceType::DeviceCUDA, gate, up), run_swiglu(DeviceType::DeviceCPU, gate, up), 2.0);  // exp differs in the last bit
    std::vector<uint16_t> table = random_bf16(size_t(100) * 512, 23);
    for (int32_t token : {0, 57, 99, 1000, -1}) {
        ASSERT_TRUE(run_embedding(DeviceType::DeviceCUDA, 100, 512, table, token) ==
                    run_embedding(DeviceType::DeviceCPU, 100, 512, table, token));
    }
}

TEST_GPU(test_decode_layers, rope_cuda_matches_cpu) {
    const int n_q = 8, n_kv = 2, max_pos = 64;
    std::vector<uint16_t> qkv = random_bf16(size_t(n_q + 2 * n_kv) * 128, 31, 1.5);
    std::vector<uint16_t> qg = random_bf16(128, 32, 0.1, 1.0), kg = random_bf16(128, 33, 0.1, 1.0);
    for (int32_t pos : {0, 1, 37, 63}) {
        RopeResult gpu = run_rope(DeviceType::DeviceCUDA, n_q, n_kv, max_pos, pos, qkv, qg, kg, 1e6f, 1e-6f);
        RopeResult cpu = run_rope(DeviceType::DeviceCPU, n_q, n_kv, max_pos, pos, qkv, qg, kg, 1e6f, 1e-6f);
        // sin/cos of the two sides differ in the last bits: normalised, rotated heads are O(1) numbers, two
        // bf16 ulps of the head's scale
        for (size_t i = 0; i < gpu.q.size(); i++) ASSERT_LE(std::fabs(fl(gpu.q[i]) - fl(cpu.q[i])), 0.0625);
        for (size_t i = 0; i < gpu.k_cache.size(); i++) ASSERT_LE(std::fabs(fl(gpu.k_cache[i]) - fl(cpu.k_cache[i])), 0.0625);
        ASSERT_TRUE(gpu.v_cache == cpu.v_cache);
    }
}

TEST_GPU(test_decode_layers, mha_cuda_matches_cpu) {
    struct Case { int n_q, n_kv, max_pos, pos; };
    for (const Case& c : {Case{8, 2, 200, 150}, Case{4, 4, 64, 0}, Case{16, 2, 130, 129}, Case{2, 1, 64, 63}}) {
        std::vector<uint16_t> q = random_bf16(size_t(c.n_q) * 128, 41), kc = random_bf16(size_t(c.max_pos) * c.n_kv * 128, 42);
        std::vector<uint16_t> vc = random_bf16(kc.size(), 43);
        std::vector<uint16_t> gpu = run_mha(DeviceType::DeviceCUDA, c.n_q, c.n_kv, c.max_pos, c.pos, q, kc, vc);
        std::vector<uint16_t> cpu = run_mha(DeviceType::DeviceCPU, c.n_q, c.n_kv, c.max_pos, c.pos, q, kc, vc);
        double num = 0, den = 0;
        for (size_t i = 0; i < gpu.size(); i++) {
            ASSERT_TRUE(std::isfinite(fl(gpu[i])));
            num += (fl(gpu[i]) - fl(cpu[i])) * (fl(gpu[i]) - fl(cpu[i]));
            den += fl(cpu[i]) * fl(cpu[i]);
        }
        ASSERT_LE(std::sqrt(num / den), 4e-3);  // one bf16 rounding of the output on each side
    }
}
