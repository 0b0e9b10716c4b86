// Host side of the fused INT4 AWQ dequantise + GEMV: shape checks, launch plan, C ABI.
#include "kx_awq_gemv_kernel.h"

namespace kx {
namespace {

struct AwqPlan {
    int waves;     // waves per workgroup stacked along K (4, 8 or 16)
    int rt;        // consecutive rows per lane (8 or 16)
    int mb;        // activation rows per workgroup (1, 2, 4 or 8)
    int coltiles;  // tiles of 256 output columns
    int ktiles;    // workgroups along K that share a column tile
    int mtiles;    // ceil(M / mb)
};

inline int rows_per_block(int waves, int rt) {
    return waves * kSlotsPerWave * rt;
}

inline AwqPlan make_plan(int M, int K, int N) {
    AwqPlan p;
    p.mb = M >= 8 ? 8 : (M >= 4 ? 4 : (M >= 2 ? 2 : 1));
    p.mtiles = (M + p.mb - 1) / p.mb;
    p.coltiles = (N / 8 + kWC - 1) / kWC;
    // Eight waves of sixteen rows per lane (256 rows of K per workgroup) measured best or within
    // noise of best on every Qwen3 projection shape; shorter K takes fewer waves so that no
    // workgroup is mostly idle.
    p.rt = 16;
    p.waves = 8;
    while (p.waves > 4 && rows_per_block(p.waves, p.rt) > K) p.waves /= 2;
    if (rows_per_block(p.waves, p.rt) > K) p.rt = 8;
    const int kb = rows_per_block(p.waves, p.rt);
    p.ktiles = (K + kb - 1) / kb;
    return p;
}

template <int WAVES, int RT>
void launch_mb(const AwqPlan& p, const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
               const int32_t* qzeros, uint16_t* y, float* partials, uint32_t* counters, int M,
               int K, int N, int group, hipStream_t stream) {
#define KX_ARGS x, qweight, scales, qzeros, y, partials, counters, M, K, N, group, p.coltiles, p.ktiles, p.mtiles, stream
    switch (p.mb) {
        case 1: launch_awq_gemv<WAVES, RT, 1>(KX_ARGS); break;
        case 2: launch_awq_gemv<WAVES, RT, 2>(KX_ARGS); break;
        case 4: launch_awq_gemv<WAVES, RT, 4>(KX_ARGS); break;
        default: launch_awq_gemv<WAVES, RT, 8>(KX_ARGS); break;
    }
#undef KX_ARGS
}

__global__ void fill_zero_u32(uint32_t* p, size_t n) {
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

}  // namespace
}  // namespace kx

extern "C" size_t kx_gemv_workspace_bytes(int32_t M, int32_t K, int32_t N) {
    if (M < 1 || M > KX_MAX_BATCH || K < 1 || N < 8) return 0;
    const kx::AwqPlan p = kx::make_plan(M, K, N);
    return kx::kCounterBytes + static_cast<size_t>(p.ktiles) * M * static_cast<size_t>(N) * sizeof(float);
}

extern "C" int kx_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
    if (!workspace) return KX_ERR_NULL_POINTER;
    if (workspace_bytes < kx::kCounterBytes) return KX_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) % 256) return KX_ERR_ALIGNMENT;
    // A fill kernel rather than hipMemsetAsync, so that the call may sit inside a captured graph.
    size_t n = kx::kCounterBytes / sizeof(uint32_t);
    hipLaunchKernelGGL(kx::fill_zero_u32, dim3((n + 255) / 256), dim3(256), 0, kx::as_stream(stream),
                       static_cast<uint32_t*>(workspace), n);
    return kx::launch_status();
}

extern "C" int kx_gemv_awq_bf16(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                                const int32_t* qzeros, uint16_t* y, int32_t M, int32_t K, int32_t N,
                                int32_t group_size, void* workspace, size_t workspace_bytes,
                                void* stream) {
    if (!x || !qweight || !scales || !qzeros || !y) return KX_ERR_NULL_POINTER;
    if (M < 1 || M > KX_MAX_BATCH || K < 1 || N < 8 || (N % 8) != 0) return KX_ERR_BAD_SHAPE;
    if (group_size < 32 || (group_size % 32) != 0 || (K % group_size) != 0) return KX_ERR_BAD_SHAPE;
    if (reinterpret_cast<uintptr_t>(scales) % 16 || reinterpret_cast<uintptr_t>(x) % 16 ||
        reinterpret_cast<uintptr_t>(qweight) % 4 || reinterpret_cast<uintptr_t>(qzeros) % 4 ||
        reinterpret_cast<uintptr_t>(y) % 8) {
        return KX_ERR_ALIGNMENT;
    }
    kx::AwqPlan p = kx::make_plan(M, K, N);
    float* partials = nullptr;
    uint32_t* counters = nullptr;
    if (p.ktiles > 1) {
        if (!workspace) return KX_ERR_WORKSPACE;
        if (reinterpret_cast<uintptr_t>(workspace) % 256) return KX_ERR_ALIGNMENT;
        size_t need = kx::kCounterBytes + static_cast<size_t>(p.ktiles) * M * N * sizeof(float);
        if (workspace_bytes < need) return KX_ERR_WORKSPACE;
        if (p.coltiles * p.mtiles > kx::kMaxTiles) return KX_ERR_BAD_SHAPE;
        counters = static_cast<uint32_t*>(workspace);
        partials = reinterpret_cast<float*>(static_cast<char*>(workspace) + kx::kCounterBytes);
    }
    hipStream_t s = kx::as_stream(stream);
#define KX_ARGS p, x, qweight, scales, qzeros, y, partials, counters, M, K, N, group_size, s
    if (p.waves == 8) {
        kx::launch_mb<8, 16>(KX_ARGS);
    } else if (p.rt == 16) {
        kx::launch_mb<4, 16>(KX_ARGS);
    } else {
        kx::launch_mb<4, 8>(KX_ARGS);
    }
#undef KX_ARGS
    return kx::launch_status();
}
