// GPU side of the matmul operator: tensors in, C ABI out.
#include "matmul_kernel.h"

#include <hip/hip_runtime_api.h>

#include <map>
#include <memory>

#include "../kernel_interface.h"
#include "kx_hip.h"

namespace kernel {
namespace {

struct Workspace {
    std::shared_ptr<base::Buffer> buffer;
};

// One workspace per stream: launches on one stream run in order and may share it, launches on
// different streams may overlap and must not.  Single host thread assumed, like the rest of the
// host API.
std::map<void*, Workspace>& workspaces() {
    static std::map<void*, Workspace> table;
    return table;
}

bool stream_is_capturing(void* stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &status) != hipSuccess) {
        (void)hipGetLastError();  // a stream that cannot be asked is treated as not capturing
        return false;
    }
    return status != hipStreamCaptureStatusNone;
}

// The C ABI's structs carry no size field: a library built from another version of kx_hip.h would read other
// fields, so the first call through this file compares versions.
void check_abi_once() {
    static const bool checked = [] {
        CHECK_EQ(kx_abi_version(), KX_ABI_VERSION) << "libkx_hip.so and this build of the host API disagree about kx_hip.h";
        return true;
    }();
    (void)checked;
}

void* workspace_for(void* stream, size_t bytes) {
    check_abi_once();
    if (bytes == 0) {
        return nullptr;
    }
    Workspace& ws = workspaces()[stream];
    if (ws.buffer == nullptr || ws.buffer->byte_size() < bytes) {
        // Growing means allocating, waiting for the stream and initialising counters: none of that may
        // happen while the stream records a graph (it would be refused, or end up inside the graph).
        CHECK(!stream_is_capturing(stream))
            << "the matmul workspace of this stream must grow to " << bytes
            << " bytes while the stream is capturing: call kernel::matmul_reserve_workspace(stream, M, K, N) "
               "for the largest projection before the capture begins";
        if (ws.buffer != nullptr) {
            // the old buffer may still be in use by launches already enqueued on this stream
            (void)hipStreamSynchronize(static_cast<hipStream_t>(stream));
        }
        ws.buffer = std::make_shared<base::Buffer>(bytes, base::CUDADeviceAllocatorFactory::get_instance());
        CHECK_NE(ws.buffer->ptr(), nullptr);
        const int rc = kx_workspace_init(ws.buffer->ptr(), bytes, stream);
        CHECK_EQ(rc, KX_OK) << "workspace init failed: " << kx_error_string(rc);
    }
    return ws.buffer->ptr();
}

int32_t rows_of(const tensor::Tensor& t, int32_t inner) {
    if (t.dims_size() == 1) {
        CHECK_EQ(t.get_dim(0), inner);
        return 1;
    }
    CHECK_EQ(t.dims_size(), 2);
    CHECK_EQ(t.get_dim(1), inner);
    return t.get_dim(0);
}

}  // namespace

void matmul_release_workspaces() {
    workspaces().clear();
}

void matmul_release_workspace(void* stream) {
    auto it = workspaces().find(stream);
    if (it == workspaces().end()) return;
    // The allocator hands a released block to the next request at once, and that request zeroes its counters:
    // launches still queued on this stream must have finished with the block before it goes back.  A stream
    // that records a graph cannot be waited for; its block stays in the table until matmul_release_workspaces().
    if (stream_is_capturing(stream)) {
        LOG(ERROR) << "the matmul workspace of a capturing stream is kept until matmul_release_workspaces()";
        return;
    }
    if (it->second.buffer != nullptr) {
        const hipError_t err = hipStreamSynchronize(static_cast<hipStream_t>(stream));
        if (err != hipSuccess) {
            (void)hipGetLastError();
            LOG(ERROR) << "could not wait for the stream before releasing its matmul workspace: "
                       << hipGetErrorString(err);
        }
    }
    workspaces().erase(it);
}

void matmul_reserve_workspace(void* stream, int32_t M, int32_t K, int32_t N) {
    (void)workspace_for(stream, kx_gemv_workspace_bytes(M, K, N));
}

void matmul_kernel_cu(const tensor::Tensor& input, const tensor::Tensor& weight,
                      const tensor::Tensor& output, void* stream) {
    CHECK(input.device_type() == base::DeviceType::DeviceCUDA);
    CHECK(weight.device_type() == base::DeviceType::DeviceCUDA);
    CHECK(output.device_type() == base::DeviceType::DeviceCUDA);
    CHECK_EQ(input.is_empty(), false);
    CHECK_EQ(weight.is_empty(), false);
    CHECK_EQ(output.is_empty(), false);
    CHECK_EQ(weight.dims_size(), 2);
    const int32_t N = weight.get_dim(0);
    const int32_t K = weight.get_dim(1);
    const int32_t M = rows_of(input, K);
    CHECK_EQ(rows_of(output, N), M);

    const int rc = kx_gemv_bf16(input.ptr<uint16_t>(), weight.ptr<uint16_t>(),
                                const_cast<uint16_t*>(output.ptr<uint16_t>()), M, K, N, nullptr, 0, stream);
    CHECK(rc == KX_OK) << "BF16 matmul kernel launch failed: " << kx_error_string(rc);
}

void matmul_kernel_awq_cu(const tensor::Tensor& input, const tensor::Tensor& qweight,
                          const tensor::Tensor& scales, const tensor::Tensor& qzeros,
                          const tensor::Tensor& output, int32_t group_size, void* stream) {
    CHECK(input.device_type() == base::DeviceType::DeviceCUDA);
    CHECK(qweight.device_type() == base::DeviceType::DeviceCUDA);
    CHECK(scales.device_type() == base::DeviceType::DeviceCUDA);
    CHECK(qzeros.device_type() == base::DeviceType::DeviceCUDA);
    CHECK(output.device_type() == base::DeviceType::DeviceCUDA);
    CHECK_EQ(input.is_empty(), false);
    CHECK_EQ(qweight.is_empty(), false);
    CHECK_EQ(scales.is_empty(), false);
    CHECK_EQ(qzeros.is_empty(), false);
    CHECK_EQ(output.is_empty(), false);
    CHECK_EQ(qweight.dims_size(), 2);
    CHECK_GT(group_size, 0);
    const int32_t K = qweight.get_dim(0);
    const int32_t N = qweight.get_dim(1) * 8;
    CHECK_EQ(K % group_size, 0);
    CHECK_EQ(scales.size(), static_cast<size_t>(K / group_size) * N);
    CHECK_EQ(qzeros.size(), static_cast<size_t>(K / group_size) * (N / 8));
    const int32_t M = rows_of(input, K);
    CHECK_EQ(rows_of(output, N), M);

    const size_t ws_bytes = kx_gemv_workspace_bytes(M, K, N);
    void* ws = workspace_for(stream, ws_bytes);
    const int rc = kx_gemv_awq_bf16(input.ptr<uint16_t>(), qweight.ptr<int32_t>(), scales.ptr<uint16_t>(),
                                    qzeros.ptr<int32_t>(), const_cast<uint16_t*>(output.ptr<uint16_t>()), M, K,
                                    N, group_size, ws, ws_bytes, stream);
    CHECK(rc == KX_OK) << "AWQ matmul kernel launch failed: " << kx_error_string(rc);
}

namespace {

void expect_gpu_tensor(const tensor::Tensor& t, const char* what) {
    CHECK_EQ(t.is_empty(), false) << what;
    CHECK(t.device_type() == base::DeviceType::DeviceCUDA) << what;
}

uint16_t* u16_of(const tensor::Tensor& t) {
    return const_cast<uint16_t*>(t.ptr<uint16_t>());
}

}  // namespace

void matmul_chain_kernel_cu(const MatmulChain& chain, const tensor::Tensor& qweight, const tensor::Tensor& scales,
                            const tensor::Tensor& qzeros, int32_t group_size, void* stream) {
    expect_gpu_tensor(qweight, "qweight");
    expect_gpu_tensor(scales, "scales");
    expect_gpu_tensor(qzeros, "qzeros");
    CHECK_EQ(qweight.dims_size(), 2);
    CHECK_GT(group_size, 0);
    const int32_t K = qweight.get_dim(0);
    const int32_t N = qweight.get_dim(1) * 8;
    CHECK_EQ(K % group_size, 0);
    CHECK_EQ(scales.size(), static_cast<size_t>(K / group_size) * N);
    CHECK_EQ(qzeros.size(), static_cast<size_t>(K / group_size) * (N / 8));

    kx_chain_desc d{};
    switch (chain.in) {
        case MatmulChain::In::Row:
            expect_gpu_tensor(chain.x, "activation row");
            CHECK_EQ(chain.x.size(), static_cast<size_t>(K));
            d.in_kind = KX_IN_ROW;
            d.x = chain.x.ptr<uint16_t>();
            break;
        case MatmulChain::In::SwiGLU:
            expect_gpu_tensor(chain.gate, "gate");
            expect_gpu_tensor(chain.up, "up");
            CHECK_EQ(chain.gate.size(), static_cast<size_t>(K));
            CHECK_EQ(chain.up.size(), static_cast<size_t>(K));
            d.in_kind = KX_IN_SWIGLU;
            d.gate = chain.gate.ptr<uint16_t>();
            d.up = chain.up.ptr<uint16_t>();
            break;
        case MatmulChain::In::AttentionChunks:
            expect_gpu_tensor(chain.attention_chunks, "attention chunks");
            d.in_kind = KX_IN_ATTN;
            d.attn_workspace = chain.attention_chunks.ptr<uint8_t>();
            d.attn_workspace_bytes = chain.attention_chunks.byte_size();
            d.n_q_heads = chain.n_q_heads;
            d.n_kv_heads = chain.n_kv_heads;
            d.max_positions = chain.max_positions;
            break;
        case MatmulChain::In::NormFromTileSums:
            expect_gpu_tensor(chain.norm_row, "row to normalise");
            expect_gpu_tensor(chain.norm_tile_sumsq, "tile sums of squares");
            expect_gpu_tensor(chain.norm_gain, "norm gain");
            CHECK_EQ(chain.norm_row.size(), static_cast<size_t>(K));
            CHECK_EQ(chain.norm_gain.size(), static_cast<size_t>(K));
            CHECK_EQ(chain.norm_tile_sumsq.size(), static_cast<size_t>((K + 255) / 256) * 4);
            d.in_kind = KX_IN_NORM;
            d.norm_row = chain.norm_row.ptr<uint16_t>();
            d.norm_sumsq = chain.norm_tile_sumsq.ptr<float>();
            d.norm_parts = (K + 255) / 256;
            d.norm_gain = chain.norm_gain.ptr<uint16_t>();
            d.norm_eps = chain.norm_eps;
            break;
    }
    switch (chain.out) {
        case MatmulChain::Out::Row:
            expect_gpu_tensor(chain.y, "output row");
            CHECK_EQ(chain.y.size(), static_cast<size_t>(N));
            d.out_kind = KX_OUT_ROW;
            d.y = u16_of(chain.y);
            break;
        case MatmulChain::Out::Residual:
            expect_gpu_tensor(chain.residual, "residual row");
            expect_gpu_tensor(chain.tile_sumsq, "tile sums of squares");
            CHECK_EQ(chain.residual.size(), static_cast<size_t>(N));
            CHECK_EQ(chain.tile_sumsq.size(), static_cast<size_t>((N + 255) / 256) * 4);
            d.out_kind = KX_OUT_RESIDUAL;
            d.residual_in = chain.residual.ptr<uint16_t>();
            d.residual_out = u16_of(chain.residual);
            d.sumsq_out = const_cast<float*>(chain.tile_sumsq.ptr<float>());
            break;
        case MatmulChain::Out::QkvRope:
            expect_gpu_tensor(chain.q_gain, "q gain");
            expect_gpu_tensor(chain.k_gain, "k gain");
            expect_gpu_tensor(chain.q_out, "q output");
            expect_gpu_tensor(chain.k_cache, "key cache");
            expect_gpu_tensor(chain.v_cache, "value cache");
            expect_gpu_tensor(chain.pos, "position");
            CHECK_EQ(chain.k_cache.dims_size(), 3);
            CHECK_EQ(chain.v_cache.size(), chain.k_cache.size());
            d.out_kind = KX_OUT_QKV_ROPE;
            d.q_gain = chain.q_gain.ptr<uint16_t>();
            d.k_gain = chain.k_gain.ptr<uint16_t>();
            d.q_out = u16_of(chain.q_out);
            d.k_cache = u16_of(chain.k_cache);
            d.v_cache = u16_of(chain.v_cache);
            d.pos = chain.pos.ptr<int32_t>();
            d.rope_n_q_heads = chain.rope_n_q_heads;
            d.rope_n_kv_heads = chain.rope_n_kv_heads;
            d.cache_positions = chain.k_cache.get_dim(0);
            d.rope_theta = chain.rope_theta;
            d.qk_eps = chain.qk_eps;
            break;
    }
    const size_t ws_bytes = kx_gemv_workspace_bytes(1, K, N);
    void* ws = workspace_for(stream, ws_bytes);
    const int rc = kx_gemv_awq_chain_bf16(&d, qweight.ptr<int32_t>(), scales.ptr<uint16_t>(), qzeros.ptr<int32_t>(), K, N,
                                          group_size, ws, ws_bytes, stream);
    CHECK(rc == KX_OK) << "fused AWQ matmul launch failed: " << kx_error_string(rc);
}

}  // namespace kernel
