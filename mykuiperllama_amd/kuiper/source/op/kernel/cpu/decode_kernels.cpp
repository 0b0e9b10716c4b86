// Host kernels of the decode-step operators (explicit DeviceCPU layers only).
#include "decode_kernels.h"

#include <cmath>
#include <vector>

#include "bf16.h"

namespace kernel {
namespace {

constexpr int32_t kHeadDim = 128;

void expect_cpu(const tensor::Tensor& t) {
    CHECK_EQ(t.is_empty(), false);
    CHECK(t.device_type() == base::DeviceType::DeviceCPU);
}

}  // namespace

void rmsnorm_kernel_cpu(const tensor::Tensor& input, const tensor::Tensor& delta, const tensor::Tensor& weight,
                        const tensor::Tensor& output, float eps, void* stream) {
    UNUSED(stream);
    expect_cpu(input);
    expect_cpu(weight);
    expect_cpu(output);
    const int32_t n = static_cast<int32_t>(weight.size());
    CHECK_GT(n, 0);
    CHECK_EQ(input.size() % n, size_t(0));
    CHECK_EQ(input.size(), output.size());
    const bool add = !delta.is_empty();
    if (add) {
        expect_cpu(delta);
        CHECK_EQ(delta.size(), input.size());
    }
    uint16_t* x = const_cast<uint16_t*>(input.ptr<uint16_t>());
    const uint16_t* d = add ? delta.ptr<uint16_t>() : nullptr;
    const uint16_t* g = weight.ptr<uint16_t>();
    uint16_t* y = const_cast<uint16_t*>(output.ptr<uint16_t>());
    const size_t rows = input.size() / n;
    for (size_t r = 0; r < rows; r++) {
        float ss = 0.0f;
        for (int32_t i = 0; i < n; i++) {
            const size_t at = r * n + i;
            if (add) x[at] = float_to_bf16(bf16_to_float(x[at]) + bf16_to_float(d[at]));  // the residual add, in place
            const float v = bf16_to_float(x[at]);
            ss += v * v;
        }
        const float inv = 1.0f / std::sqrt(ss / static_cast<float>(n) + eps);
        for (int32_t i = 0; i < n; i++) {
            const size_t at = r * n + i;
            y[at] = float_to_bf16(bf16_to_float(g[i]) * round_bf16(bf16_to_float(x[at]) * inv));
        }
    }
}

void swiglu_kernel_cpu(const tensor::Tensor& gate, const tensor::Tensor& up, const tensor::Tensor& output,
                       void* stream) {
    UNUSED(stream);
    expect_cpu(gate);
    expect_cpu(up);
    expect_cpu(output);
    CHECK_EQ(gate.size(), up.size());
    CHECK_EQ(gate.size(), output.size());
    const uint16_t* g = gate.ptr<uint16_t>();
    const uint16_t* u = up.ptr<uint16_t>();
    uint16_t* y = const_cast<uint16_t*>(output.ptr<uint16_t>());
    for (size_t i = 0; i < gate.size(); i++) {
        const float gv = bf16_to_float(g[i]);
        const float act = round_bf16(gv / (1.0f + std::exp(-gv)));  // silu(g) is a bf16 tensor before it meets up
        y[i] = float_to_bf16(act * bf16_to_float(u[i]));
    }
}

void embedding_kernel_cpu(const tensor::Tensor& token, const tensor::Tensor& table, const tensor::Tensor& output,
                          void* stream) {
    UNUSED(stream);
    expect_cpu(token);
    expect_cpu(table);
    expect_cpu(output);
    CHECK_EQ(table.dims_size(), 2);
    const int32_t vocab = table.get_dim(0);
    const int32_t dim = table.get_dim(1);
    CHECK_EQ(output.size(), static_cast<size_t>(dim));
    int32_t t = token.ptr<int32_t>()[0];
    t = t < 0 ? 0 : (t >= vocab ? vocab - 1 : t);
    const uint16_t* row = table.ptr<uint16_t>() + static_cast<size_t>(t) * dim;
    uint16_t* y = const_cast<uint16_t*>(output.ptr<uint16_t>());
    for (int32_t i = 0; i < dim; i++) y[i] = row[i];
}

void rope_kernel_cpu(const tensor::Tensor& qkv, const tensor::Tensor& q_gain, const tensor::Tensor& k_gain,
                     const tensor::Tensor& pos, const tensor::Tensor& q_out, const tensor::Tensor& k_cache,
                     const tensor::Tensor& v_cache, int32_t n_q_heads, int32_t n_kv_heads, float theta, float eps,
                     void* stream) {
    UNUSED(stream);
    expect_cpu(qkv);
    expect_cpu(q_gain);
    expect_cpu(k_gain);
    expect_cpu(pos);
    expect_cpu(q_out);
    expect_cpu(k_cache);
    expect_cpu(v_cache);
    const int32_t heads = n_q_heads + 2 * n_kv_heads;
    CHECK_EQ(qkv.size(), static_cast<size_t>(heads) * kHeadDim);
    CHECK_EQ(q_out.size(), static_cast<size_t>(n_q_heads) * kHeadDim);
    const int32_t p = pos.ptr<int32_t>()[0];
    CHECK_GE(p, 0);
    CHECK_LT(static_cast<size_t>(p) * n_kv_heads * kHeadDim, k_cache.size());
    const uint16_t* src = qkv.ptr<uint16_t>();
    uint16_t* q = const_cast<uint16_t*>(q_out.ptr<uint16_t>());
    uint16_t* kc = const_cast<uint16_t*>(k_cache.ptr<uint16_t>());
    uint16_t* vc = const_cast<uint16_t*>(v_cache.ptr<uint16_t>());
    const float log2_theta = std::log2(theta);
    for (int32_t h = 0; h < heads; h++) {
        const uint16_t* x = src + static_cast<size_t>(h) * kHeadDim;
        if (h >= n_q_heads + n_kv_heads) {  // value head: straight into the cache
            uint16_t* dst = vc + (static_cast<size_t>(p) * n_kv_heads + (h - n_q_heads - n_kv_heads)) * kHeadDim;
            for (int32_t i = 0; i < kHeadDim; i++) dst[i] = x[i];
            continue;
        }
        const bool is_q = h < n_q_heads;
        const uint16_t* gain = is_q ? q_gain.ptr<uint16_t>() : k_gain.ptr<uint16_t>();
        float ss = 0.0f;
        for (int32_t i = 0; i < kHeadDim; i++) ss += bf16_to_float(x[i]) * bf16_to_float(x[i]);
        const float inv = 1.0f / std::sqrt(ss / static_cast<float>(kHeadDim) + eps);
        float normed[kHeadDim];
        for (int32_t i = 0; i < kHeadDim; i++) {
            normed[i] = round_bf16(bf16_to_float(gain[i]) * round_bf16(bf16_to_float(x[i]) * inv));
        }
        uint16_t* dst = is_q ? q + static_cast<size_t>(h) * kHeadDim
                             : kc + (static_cast<size_t>(p) * n_kv_heads + (h - n_q_heads)) * kHeadDim;
        for (int32_t i = 0; i < kHeadDim / 2; i++) {  // rotate-half convention: partners i and i + 64
            const float freq = std::exp2(-log2_theta * static_cast<float>(i) / 64.0f);
            const float angle = static_cast<float>(p) * freq;
            const float c = std::cos(angle), s = std::sin(angle);
            dst[i] = float_to_bf16(normed[i] * c - normed[i + 64] * s);
            dst[i + 64] = float_to_bf16(normed[i + 64] * c + normed[i] * s);
        }
    }
}

void mha_kernel_cpu(const tensor::Tensor& q, const tensor::Tensor& k_cache, const tensor::Tensor& v_cache,
                    const tensor::Tensor& pos, const tensor::Tensor& workspace, const tensor::Tensor& output,
                    int32_t n_q_heads, int32_t n_kv_heads, void* stream) {
    UNUSED(stream);
    UNUSED(workspace);
    expect_cpu(q);
    expect_cpu(k_cache);
    expect_cpu(v_cache);
    expect_cpu(pos);
    expect_cpu(output);
    CHECK_EQ(q.size(), static_cast<size_t>(n_q_heads) * kHeadDim);
    CHECK_EQ(output.size(), q.size());
    CHECK_EQ(n_q_heads % n_kv_heads, 0);
    const int32_t group = n_q_heads / n_kv_heads;
    const int32_t p = pos.ptr<int32_t>()[0];
    CHECK_GE(p, 0);
    CHECK_LT(static_cast<size_t>(p) * n_kv_heads * kHeadDim, k_cache.size());
    const uint16_t* qp = q.ptr<uint16_t>();
    const uint16_t* kc = k_cache.ptr<uint16_t>();
    const uint16_t* vc = v_cache.ptr<uint16_t>();
    uint16_t* out = const_cast<uint16_t*>(output.ptr<uint16_t>());
    const float scale = 1.0f / std::sqrt(static_cast<float>(kHeadDim));
    std::vector<float> score(static_cast<size_t>(p) + 1);
    for (int32_t h = 0; h < n_q_heads; h++) {
        const int32_t kvh = h / group;
        float top = -INFINITY;
        for (int32_t t = 0; t <= p; t++) {
            const uint16_t* krow = kc + (static_cast<size_t>(t) * n_kv_heads + kvh) * kHeadDim;
            float dot = 0.0f;
            for (int32_t i = 0; i < kHeadDim; i++) dot += bf16_to_float(qp[h * kHeadDim + i]) * bf16_to_float(krow[i]);
            score[t] = dot * scale;
            top = std::fmax(top, score[t]);
        }
        float total = 0.0f;
        for (int32_t t = 0; t <= p; t++) {
            score[t] = std::exp(score[t] - top);
            total += score[t];
        }
        float acc[kHeadDim] = {0.0f};
        for (int32_t t = 0; t <= p; t++) {
            const uint16_t* vrow = vc + (static_cast<size_t>(t) * n_kv_heads + kvh) * kHeadDim;
            for (int32_t i = 0; i < kHeadDim; i++) acc[i] += score[t] * bf16_to_float(vrow[i]);
        }
        for (int32_t i = 0; i < kHeadDim; i++) out[h * kHeadDim + i] = float_to_bf16(acc[i] / total);
    }
}

}  // namespace kernel
