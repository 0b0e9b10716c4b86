// GPU wrappers of the decode-step operators over the C ABI (include/kx_hip.h).
#include "decode_kernels.h"

#include "kx_hip.h"

namespace kernel {
namespace {

constexpr int32_t kHeadDim = 128;

void expect_gpu(const tensor::Tensor& t) {
    CHECK_EQ(t.is_empty(), false);
    CHECK(t.device_type() == base::DeviceType::DeviceCUDA);
}

uint16_t* out_ptr(const tensor::Tensor& t) {
    return const_cast<uint16_t*>(t.ptr<uint16_t>());
}

}  // namespace

void rmsnorm_kernel_cu(const tensor::Tensor& input, const tensor::Tensor& delta, const tensor::Tensor& weight,
                       const tensor::Tensor& output, float eps, void* stream) {
    expect_gpu(input);
    expect_gpu(weight);
    expect_gpu(output);
    const int32_t n = static_cast<int32_t>(weight.size());
    CHECK_GT(n, 0);
    CHECK_EQ(input.size() % n, size_t(0));
    CHECK_EQ(input.size(), output.size());
    const int32_t rows = static_cast<int32_t>(input.size() / n);
    int rc;
    if (delta.is_empty()) {
        rc = kx_rmsnorm_bf16(input.ptr<uint16_t>(), weight.ptr<uint16_t>(), out_ptr(output), rows, n, eps, stream);
    } else {
        expect_gpu(delta);
        CHECK_EQ(delta.size(), input.size());
        rc = kx_add_rmsnorm_bf16(out_ptr(input), delta.ptr<uint16_t>(), weight.ptr<uint16_t>(), out_ptr(output), rows,
                                 n, eps, stream);
    }
    CHECK(rc == KX_OK) << "RMSNorm kernel launch failed: " << kx_error_string(rc);
}

void swiglu_kernel_cu(const tensor::Tensor& gate, const tensor::Tensor& up, const tensor::Tensor& output,
                      void* stream) {
    expect_gpu(gate);
    expect_gpu(up);
    expect_gpu(output);
    CHECK_EQ(gate.size(), up.size());
    CHECK_EQ(gate.size(), output.size());
    const int rc = kx_swiglu_bf16(gate.ptr<uint16_t>(), up.ptr<uint16_t>(), out_ptr(output),
                                  static_cast<int32_t>(gate.size()), stream);
    CHECK(rc == KX_OK) << "SwiGLU kernel launch failed: " << kx_error_string(rc);
}

void embedding_kernel_cu(const tensor::Tensor& token, const tensor::Tensor& table, const tensor::Tensor& output,
                         void* stream) {
    expect_gpu(token);
    expect_gpu(table);
    expect_gpu(output);
    CHECK_EQ(table.dims_size(), 2);
    CHECK_EQ(output.size(), static_cast<size_t>(table.get_dim(1)));
    const int rc = kx_embedding_bf16(table.ptr<uint16_t>(), token.ptr<int32_t>(), out_ptr(output), table.get_dim(0),
                                     table.get_dim(1), stream);
    CHECK(rc == KX_OK) << "embedding kernel launch failed: " << kx_error_string(rc);
}

void rope_kernel_cu(const tensor::Tensor& qkv, const tensor::Tensor& q_gain, const tensor::Tensor& k_gain,
                    const tensor::Tensor& pos, const tensor::Tensor& q_out, const tensor::Tensor& k_cache,
                    const tensor::Tensor& v_cache, int32_t n_q_heads, int32_t n_kv_heads, float theta, float eps,
                    void* stream) {
    expect_gpu(qkv);
    expect_gpu(q_gain);
    expect_gpu(k_gain);
    expect_gpu(pos);
    expect_gpu(q_out);
    expect_gpu(k_cache);
    expect_gpu(v_cache);
    CHECK_EQ(qkv.size(), static_cast<size_t>(n_q_heads + 2 * n_kv_heads) * kHeadDim);
    CHECK_EQ(q_out.size(), static_cast<size_t>(n_q_heads) * kHeadDim);
    // rows of [n_kv_heads][128] the caches hold: the kernel writes no row outside them
    const size_t row = static_cast<size_t>(n_kv_heads) * kHeadDim;
    CHECK_EQ(k_cache.size(), v_cache.size());
    CHECK(k_cache.size() >= row && k_cache.size() % row == 0) << "KV cache is not [positions][n_kv_heads][128]";
    const int32_t cache_positions = static_cast<int32_t>(k_cache.size() / row);
    const int rc = kx_qk_norm_rope_bf16(qkv.ptr<uint16_t>(), q_gain.ptr<uint16_t>(), k_gain.ptr<uint16_t>(),
                                        out_ptr(q_out), out_ptr(k_cache), out_ptr(v_cache), n_q_heads, n_kv_heads,
                                        kHeadDim, pos.ptr<int32_t>(), cache_positions, theta, eps, stream);
    CHECK(rc == KX_OK) << "RoPE kernel launch failed: " << kx_error_string(rc);
}

void mha_kernel_cu(const tensor::Tensor& q, const tensor::Tensor& k_cache, const tensor::Tensor& v_cache,
                   const tensor::Tensor& pos, const tensor::Tensor& workspace, const tensor::Tensor& output,
                   int32_t n_q_heads, int32_t n_kv_heads, void* stream) {
    expect_gpu(q);
    expect_gpu(k_cache);
    expect_gpu(v_cache);
    expect_gpu(pos);
    expect_gpu(workspace);
    CHECK_EQ(q.size(), static_cast<size_t>(n_q_heads) * kHeadDim);
    CHECK_EQ(k_cache.dims_size(), 3);
    const int32_t max_positions = k_cache.get_dim(0);
    if (output.is_empty()) {  // the first stage alone: the chunks stay in the workspace for their consumer
        const int rc = kx_attn_decode_partial_bf16(q.ptr<uint16_t>(), k_cache.ptr<uint16_t>(), v_cache.ptr<uint16_t>(),
                                                   n_q_heads, n_kv_heads, kHeadDim, pos.ptr<int32_t>(), max_positions,
                                                   const_cast<uint8_t*>(workspace.ptr<uint8_t>()),
                                                   workspace.byte_size(), stream);
        CHECK(rc == KX_OK) << "attention kernel launch failed: " << kx_error_string(rc);
        return;
    }
    expect_gpu(output);
    CHECK_EQ(output.size(), q.size());
    const int rc = kx_attn_decode_bf16(q.ptr<uint16_t>(), k_cache.ptr<uint16_t>(), v_cache.ptr<uint16_t>(),
                                       out_ptr(output), n_q_heads, n_kv_heads, kHeadDim, pos.ptr<int32_t>(),
                                       max_positions, const_cast<uint8_t*>(workspace.ptr<uint8_t>()),
                                       workspace.byte_size(), stream);
    CHECK(rc == KX_OK) << "attention kernel launch failed: " << kx_error_string(rc);
}

}  // namespace kernel
