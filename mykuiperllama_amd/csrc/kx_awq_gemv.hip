// Host side of the fused INT4 AWQ dequantise + GEMV: shape checks, launch plan, C ABI.
#include "kx_awq_gemv_kernel.h"
#include "kx_awq_gemv_mfma_kernel.h"
#include "kx_internal.h"

#include <mutex>


namespace kx {
namespace {

struct AwqPlan {
    bool mfma;     // matrix-core kernel (any M) or the VALU kernel
    int waves;     // waves per workgroup stacked along K (4, 8 or 16)
    int rt;        // VALU kernel: consecutive rows per lane (8 or 16); MFMA kernel: 32-row steps per wave
    int mb;        // activation rows per workgroup (1, 2, 4 or 8)
    int coltiles;  // tiles of 256 output columns
    int ktiles;    // workgroups along K that share a column tile
    int mtiles;    // ceil(M / mb)
};

inline int rows_per_block(int waves, int rt) {
    return waves * kSlotsPerWave * rt;
}

constexpr int kComputeUnits = 256;  // MI355X
constexpr int kExchangeRows = 8;    // what a K tile's share of the split-K exchange costs, in rows of K streamed

inline bool is_pow2(int v) {
    return v > 0 && (v & (v - 1)) == 0;
}

// MFMA kernel: four waves per workgroup, each walking `ks` consecutive 32-row steps that must lie in
// one quantisation group.  Measured on the Qwen3-8B shapes: two steps per wave (256 rows per
// workgroup) are best up to M = 8, except that long K (down 12288 -> 4096, 48 K tiles) does better
// with four steps from M = 5 (15.7 -> 14.4 us at M = 8); from M = 9 four steps (512 rows, half the
// partial sums to exchange) win everywhere (M = 16: q 12.1 -> 10.5, gate 15.6 -> 13.7, down
// 24.7 -> 18.0 us), even where they leave fewer workgroups than compute units.
inline AwqPlan make_mfma_plan(int M, int K, int N, int group) {
    AwqPlan p;
    p.mfma = true;
    p.coltiles = (N / 8 + kWC - 1) / kWC;
    p.mb = M;
    p.mtiles = 1;
    p.waves = 4;
    int ks = (M >= 9 || (M >= 5 && K >= 8192)) ? 4 : 2;
    while (ks > 1 && ks * kStepRows > group) ks /= 2;
    while (ks > 1 && p.waves * ks * kStepRows > K) ks /= 2;
    p.rt = ks;  // steps per wave
    const int kb = p.waves * ks * kStepRows;
    p.ktiles = (K + kb - 1) / kb;
    return p;
}

inline AwqPlan make_valu_plan(int M, int K, int N, bool allow_long_rows = true, bool allow_12_waves = true) {
    AwqPlan p;
    p.mfma = false;
    p.coltiles = (N / 8 + kWC - 1) / kWC;
    p.mb = M >= 8 ? 8 : (M >= 4 ? 4 : (M >= 2 ? 2 : 1));
    p.mtiles = (M + p.mb - 1) / p.mb;
    // Three shapes of workgroup: eight waves of sixteen rows per lane (256 rows of K), eight waves of
    // 32 rows per lane (512 rows, half the partial sums to exchange) and twelve waves of sixteen
    // rows (384 rows).  What a launch costs, in rows of K streamed by the busiest compute unit, is
    // the number of workgroups that compute unit gets (all of them resident together or not) times
    // the rows of a workgroup, plus about eight rows' worth per K tile for the exchange.  Measured,
    // us per launch at M = 1 (256 / 512 / 384 rows): q 4096->4096 5.7 / 6.2 / -, gate 4096->12288
    // 8.6 / 9.3 / -, q|k|v 4096->6144 6.8 / 6.6 / -, gate|up 4096->24576 15.7 / 13.8 / -, down
    // 12288->4096 10.0 / - / 9.1, 32B-shaped q|k|v 5120->10240 10.6 / 9.8 / -, o 8192->5120
    // 9.1 / 9.3 / -: the minimum of that cost picks the faster one every time.
    // (Twelve waves of 32 rows, 768 rows per workgroup and one workgroup per compute unit on down
    // 12288->4096, are faster still on the plain launch, 9.0 -> 8.6 us, but slower with the SwiGLU
    // prologue of the decode step, whose latency then has no second workgroup to hide behind.  Eight
    // waves of eight rows, 128 rows per workgroup, for projections too narrow to give every compute
    // unit a workgroup — k 4096->1024 has 64 — are slower as well, 5.07 -> 5.48 us: twice the K tiles
    // to exchange cost more than the idle compute units.)
    // Twelve waves: one activation row, plain or SwiGLU input, plain or residual output only (the
    // other prologues and epilogues are laid out for 4 or 8 waves).  Shorter K than 256 takes fewer
    // waves so that no workgroup is mostly idle.
    p.rt = 16;
    p.waves = 8;
    if (K >= rows_per_block(8, 16)) {
        const struct { int waves, rt; bool allowed; } shapes[3] = {
            {8, 16, true}, {8, 32, allow_long_rows}, {12, 16, allow_12_waves && M == 1}};
        long best = -1;
        for (const auto& c : shapes) {
            const int rows = rows_per_block(c.waves, c.rt);
            if (!c.allowed || ((c.waves != 8 || c.rt != 16) && K % rows != 0)) continue;
            const long kt = (K + rows - 1) / rows;
            const long blocks = static_cast<long>(p.coltiles) * p.mtiles * kt;
            const long cost = (blocks + kComputeUnits - 1) / kComputeUnits * rows + kExchangeRows * kt;
            if (best < 0 || cost < best) {
                best = cost;
                p.waves = c.waves;
                p.rt = c.rt;
                p.ktiles = static_cast<int>(kt);
            }
        }
        return p;
    }
    while (p.waves > 4 && rows_per_block(p.waves, p.rt) > K) p.waves /= 2;
    if (rows_per_block(p.waves, p.rt) > K) p.rt = 8;
    const int kb = rows_per_block(p.waves, p.rt);
    p.ktiles = (K + kb - 1) / kb;
    return p;
}

// One activation row, plain store, the K tiles meeting in fixed point (splitk_exchange_store_fixed): that
// exchange costs about half of the one above per K tile, which moves the choice towards smaller workgroups -
// four waves of sixteen rows (128 rows of K, 256 threads) join the candidates.  Measured, us per launch with
// 128 / 256 / 512 / 384 rows per workgroup: k 4096->1024 3.65 / 3.85 / 4.72 / -, q 4096->4096 4.47 / 4.55 /
// 5.10 / -, q|k|v 4096->6144 5.19 / 5.52 / 5.38 / -, gate 4096->12288 8.16 / 7.63 / 8.34 / -, gate|up
// 4096->24576 13.67 / 12.81 / 12.82 / -, down 12288->4096 - / 7.75 / 8.61 / 7.28, 32B-shaped o 8192->5120
// - / 7.10 / 8.03 / -.  ktiles == 1 in the result means that the exchange does not apply (a single K tile, more
// K tiles than the slot's arrival count holds, or more columns than the zeroed area has slots for).
constexpr int kFixedExchangeRows = 4;

inline AwqPlan make_fixed_plan(int K, int N) {
    AwqPlan p{};
    p.mfma = false;
    p.coltiles = (N / 8 + kWC - 1) / kWC;
    p.mb = 1;
    p.mtiles = 1;
    p.waves = 8;
    p.rt = 16;
    p.ktiles = 1;
    if (static_cast<size_t>(N) * 16 > kCounterBytes) return p;  // a slot and a mask word per column
    const struct { int waves, rt; } shapes[4] = {{8, 16}, {4, 16}, {8, 32}, {12, 16}};
    long best = -1;
    for (const auto& c : shapes) {
        const int rows = rows_per_block(c.waves, c.rt);
        if (K < rows || ((c.waves != 8 || c.rt != 16) && K % rows != 0)) continue;
        const long kt = (K + rows - 1) / rows;
        if (kt < 2 || kt > kFixedMaxKTiles) continue;
        const long blocks = static_cast<long>(p.coltiles) * kt;
        const long cost = (blocks + kComputeUnits - 1) / kComputeUnits * rows + kFixedExchangeRows * kt;
        if (best < 0 || cost < best) {
            best = cost;
            p.waves = c.waves;
            p.rt = c.rt;
            p.ktiles = static_cast<int>(kt);
        }
    }
    return p;
}

inline AwqPlan make_plan(int M, int K, int N, int group, int mode) {
    // The MFMA kernel needs quantisation groups that tile the workgroup's K range (powers of two)
    // and loads two packed words at a time (N a multiple of sixteen).
    const bool mfma_ok = is_pow2(group) && (N % 16) == 0;  // mfma_shape_ok() below
    // One activation row stays on the vector kernel: with the fixed-point exchange it is ahead of the MFMA kernel on
    // every measured shape (kx_gemv_awq_bf16_policy decides that before it comes here), and the launches with an
    // activation prologue or an epilogue live in it.
    const bool mfma = mfma_ok && (mode == KX_POLICY_MFMA || (mode == KX_POLICY_BY_SHAPE && M >= 2));
    return mfma ? make_mfma_plan(M, K, N, group) : make_valu_plan(M, K, N);
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

// Launches with an activation prologue are built for the decode step (M = 1); larger M is served
// two activation rows per workgroup.
inline AwqPlan make_fused_plan(int M, int K, int N, bool allow_12_waves) {
    AwqPlan p = make_valu_plan(M, K, N, true, allow_12_waves);
    p.mb = M >= 2 ? 2 : 1;
    p.mtiles = (M + p.mb - 1) / p.mb;
    return p;
}

// One activation row, add + RMSNorm on the way in, per-head norm + rotation + cache append on the way out.
template <int PRO>
void launch_qkv(const AwqPlan& p, const FusedInput& fi, const RopeTarget& rope, const int32_t* qweight,
                const uint16_t* scales, const int32_t* qzeros, float* partials, uint32_t* counters, int K, int N,
                int group, hipStream_t stream) {
#define KX_ARGS nullptr, qweight, scales, qzeros, nullptr, partials, counters, 1, K, N, group, p.coltiles, p.ktiles, 1, stream, fi, rope
    if (p.rt == 32) launch_awq_gemv<8, 32, 1, PRO, kEpiQkRope>(KX_ARGS);
    else if (p.waves == 8) launch_awq_gemv<8, 16, 1, PRO, kEpiQkRope>(KX_ARGS);
    else if (p.rt == 16) launch_awq_gemv<4, 16, 1, PRO, kEpiQkRope>(KX_ARGS);
    else launch_awq_gemv<4, 8, 1, PRO, kEpiQkRope>(KX_ARGS);
#undef KX_ARGS
}

template <int PRO>
void launch_fused(const AwqPlan& p, const FusedInput& fi, const int32_t* qweight, const uint16_t* scales,
                  const int32_t* qzeros, uint16_t* y, float* partials, uint32_t* counters, int M, int K,
                  int N, int group, hipStream_t stream) {
#define KX_ARGS nullptr, qweight, scales, qzeros, y, partials, counters, M, K, N, group, p.coltiles, p.ktiles, p.mtiles, stream, fi
#define KX_BY_MB(W, R)                                                  \
    do {                                                                \
        if (p.mb == 1) launch_awq_gemv<W, R, 1, PRO>(KX_ARGS);          \
        else launch_awq_gemv<W, R, 2, PRO>(KX_ARGS);                    \
    } while (0)
    if constexpr (PRO == kProSwiGLU) {
        if (p.waves == 12) {  // one activation row by construction of the plan
            launch_awq_gemv<12, 16, 1, PRO>(KX_ARGS);
            return;
        }
    }
    if (p.rt == 32) KX_BY_MB(8, 32);
    else if (p.waves == 8) KX_BY_MB(8, 16);
    else if (p.rt == 16) KX_BY_MB(4, 16);
    else KX_BY_MB(4, 8);
#undef KX_BY_MB
#undef KX_ARGS
}

// The matrix-core kernel with an activation prologue and / or the residual epilogue, 2 <= M <= 16.
template <int PRO, int EPI>
void launch_mfma_fused(const AwqPlan& p, const FusedInput& fi, const ResidualTarget& res, const uint16_t* x,
                       const int32_t* qweight, const uint16_t* scales, const int32_t* qzeros, uint16_t* y,
                       float* partials, uint32_t* counters, int M, int K, int N, int group, hipStream_t stream,
                       const RopeTarget& rope = RopeTarget{}, size_t cache_stride = 0) {
    int group_shift = 0;
    while ((1 << group_shift) < group) group_shift++;
#define KX_MARGS x, qweight, scales, qzeros, y, partials, counters, M, K, N, group_shift, p.coltiles, p.ktiles, stream, fi, res, rope, cache_stride
#define KX_MFMA_BY_M(KS)                                                             \
    do {                                                                             \
        if (M <= 2) launch_awq_gemv_mfma<4, KS, 2, 1, PRO, EPI>(KX_MARGS);           \
        else if (M <= 4) launch_awq_gemv_mfma<4, KS, 4, 1, PRO, EPI>(KX_MARGS);      \
        else if (M <= 8) launch_awq_gemv_mfma<4, KS, 8, 1, PRO, EPI>(KX_MARGS);      \
        else launch_awq_gemv_mfma<4, KS, 8, 2, PRO, EPI>(KX_MARGS);                  \
    } while (0)
    if (p.rt == 4) KX_MFMA_BY_M(4);
    else if (p.rt == 2) KX_MFMA_BY_M(2);
    else KX_MFMA_BY_M(1);
#undef KX_MFMA_BY_M
#undef KX_MARGS
}

// What the matrix-core kernel asks of a shape: quantisation groups that tile the workgroup's K range
// (powers of two) and two packed words per load (N a multiple of sixteen).
inline bool mfma_shape_ok(int N, int group) {
    return is_pow2(group) && (N % 16) == 0;
}

inline bool aligned_to(const void* p, size_t a) {
    return reinterpret_cast<uintptr_t>(p) % a == 0;
}

// Checks shared by every AWQ entry point; `x` stands for whichever tensors feed the activations.
inline int check_awq_weights(const int32_t* qweight, const uint16_t* scales, const int32_t* qzeros,
                             const uint16_t* y, int M, int K, int N, int group_size, bool stores_y = true) {
    if (!qweight || !scales || !qzeros || (stores_y && !y)) return KX_ERR_NULL_POINTER;
    if (M < 1 || M > KX_MAX_BATCH || K < 1 || N < 8 || (N % 8) != 0) return KX_ERR_BAD_SHAPE;
    if (group_size < 32 || (group_size % 32) != 0 || (K % group_size) != 0) return KX_ERR_BAD_SHAPE;
    if (reinterpret_cast<uintptr_t>(scales) % 16 || reinterpret_cast<uintptr_t>(qweight) % 4 ||
        reinterpret_cast<uintptr_t>(qzeros) % 4 || (stores_y && reinterpret_cast<uintptr_t>(y) % 8)) {
        return KX_ERR_ALIGNMENT;
    }
    return KX_OK;
}

// The launches with an activation prologue address the packed weights with 32-bit offsets.
inline bool weights_fit_buffer_loads(int K, int N) {
    return static_cast<size_t>(K) * N / 2 < (static_cast<size_t>(1) << 31);
}

// Do the byte ranges [a, a + abytes) and [b, b + bbytes) share a byte?  Null pointers overlap nothing.
inline bool ranges_overlap(const void* a, size_t abytes, const void* b, size_t bbytes) {
    if (!a || !b || abytes == 0 || bbytes == 0) return false;
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a0 < b0 + bbytes && b0 < a0 + abytes;
}

// Splits the workspace into counters and partial sums when the plan shares column tiles.
inline int resolve_workspace(const AwqPlan& p, int M, int N, void* workspace, size_t workspace_bytes,
                             float** partials, uint32_t** counters) {
    *partials = nullptr;
    *counters = nullptr;
    if (p.ktiles <= 1) return KX_OK;
    if (!workspace) return KX_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) % 256) return KX_ERR_ALIGNMENT;
    const size_t partial_bytes = static_cast<size_t>(p.ktiles) * M * N * sizeof(float);
    if (partial_bytes >= (static_cast<size_t>(1) << 32)) return KX_ERR_BAD_SHAPE;  // 32-bit offsets in the read-back
    const size_t need = kCounterBytes + partial_bytes;
    if (workspace_bytes < need) return KX_ERR_WORKSPACE;
    if (p.coltiles * p.mtiles > kMaxTiles) return KX_ERR_BAD_SHAPE;
    *counters = static_cast<uint32_t*>(workspace);
    *partials = reinterpret_cast<float*>(static_cast<char*>(workspace) + kCounterBytes);
    return KX_OK;
}

__global__ void fill_zero_u32(uint32_t* p, size_t n) {
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

}  // namespace
}  // namespace kx

extern "C" size_t kx_gemv_workspace_bytes(int32_t M, int32_t K, int32_t N) {
    if (M < 1 || M > KX_MAX_BATCH || K < 1 || N < 8) return 0;
    // Either kernel may serve a shape (the group size and M decide); size for the larger exchange.
    const int kt_valu = kx::make_valu_plan(M, K, N, true, false).ktiles;  // the entry points that keep 8 waves exchange more
    const int kt_mfma = kx::make_mfma_plan(M, K, N, 32).ktiles;  // the smallest group gives the most K tiles
    size_t ktiles = static_cast<size_t>(kt_valu > kt_mfma ? kt_valu : kt_mfma);
    if (M == 1) {
        const size_t kt_fixed = static_cast<size_t>(kx::make_fixed_plan(K, N).ktiles);  // its slow path parks partial sums there
        if (kt_fixed > ktiles) ktiles = kt_fixed;
    }
    return kx::kCounterBytes + ktiles * M * static_cast<size_t>(N) * sizeof(float);
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

// ---- the entry point that allocates nothing ----
// The split-K workspace of kx_gemv_awq_bf16_static: arrival counters, then partial sums.  Every GPU the
// library runs on holds its own copy of this array until the process ends.
namespace {

constexpr size_t kStaticPartialBytes = static_cast<size_t>(8) << 20;
constexpr size_t kStaticScratchBytes = kx::kCounterBytes + kStaticPartialBytes;
constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

struct StaticScratch {
    std::mutex mu;
    void* ptr[kMaxDevices] = {};  // device address of `scratch` on each device, null until first use there
};

StaticScratch g_static_scratch;

// Device address of the current device's copy of `scratch`; on the first call on a device the address is
// looked up and the arrival counters are zeroed on `stream` (a kernel, so that a capturing stream records
// it like any other launch).  In host code the array's name is not a device address: only the pointer
// obtained here is ever handed to a kernel.
int static_scratch_for_current_device(void** out, hipStream_t stream) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices) return KX_ERR_BAD_SHAPE;
    std::lock_guard<std::mutex> lock(g_static_scratch.mu);
    if (!g_static_scratch.ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (!p || reinterpret_cast<uintptr_t>(p) % 256) return KX_ERR_ALIGNMENT;
        const size_t n = kx::kCounterBytes / sizeof(uint32_t);
        hipLaunchKernelGGL(kx::fill_zero_u32, dim3((n + 255) / 256), dim3(256), 0, stream, static_cast<uint32_t*>(p), n);
        const int rc = kx::launch_status();
        if (rc != KX_OK) return rc;
        g_static_scratch.ptr[dev] = p;
    }
    *out = g_static_scratch.ptr[dev];
    return KX_OK;
}

}  // namespace

extern "C" size_t kx_gemv_awq_static_scratch_bytes(void) {
    return kStaticScratchBytes;
}

extern "C" int kx_gemv_awq_bf16_static(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                                       const int32_t* qzeros, uint16_t* y, int32_t M, int32_t K, int32_t N,
                                       int32_t group_size, void* stream) {
    // argument errors first, so that a rejected call touches nothing
    if (!x) return KX_ERR_NULL_POINTER;
    int rc = kx::check_awq_weights(qweight, scales, qzeros, y, M, K, N, group_size);
    if (rc != KX_OK) return rc;
    if (reinterpret_cast<uintptr_t>(x) % 16) return KX_ERR_ALIGNMENT;
    if (kx_gemv_workspace_bytes(M, K, N) > kStaticScratchBytes) return KX_ERR_WORKSPACE;  // larger than the static array
    void* ws = nullptr;
    rc = static_scratch_for_current_device(&ws, kx::as_stream(stream));
    if (rc != KX_OK) return rc;
    return kx_gemv_awq_bf16_policy(x, qweight, scales, qzeros, y, M, K, N, group_size, ws, kStaticScratchBytes, stream,
                                   KX_POLICY_BY_SHAPE);
}

extern "C" int kx_gemv_awq_bf16(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                                const int32_t* qzeros, uint16_t* y, int32_t M, int32_t K, int32_t N,
                                int32_t group_size, void* workspace, size_t workspace_bytes,
                                void* stream) {
    return kx_gemv_awq_bf16_policy(x, qweight, scales, qzeros, y, M, K, N, group_size, workspace, workspace_bytes,
                                   stream, KX_POLICY_BY_SHAPE);
}

extern "C" int kx_gemv_awq_bf16_policy(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                                       const int32_t* qzeros, uint16_t* y, int32_t M, int32_t K, int32_t N,
                                       int32_t group_size, void* workspace, size_t workspace_bytes,
                                       void* stream, int32_t policy) {
    if (policy < KX_POLICY_BY_SHAPE || policy > KX_POLICY_MFMA) return KX_ERR_BAD_SHAPE;
    if (!x) return KX_ERR_NULL_POINTER;
    int rc = kx::check_awq_weights(qweight, scales, qzeros, y, M, K, N, group_size);
    if (rc != KX_OK) return rc;
    if (reinterpret_cast<uintptr_t>(x) % 16) return KX_ERR_ALIGNMENT;
    float* partials = nullptr;
    uint32_t* counters = nullptr;
    hipStream_t s = kx::as_stream(stream);
    if (M == 1 && policy == KX_POLICY_BY_SHAPE) {
        // one activation row, plain store: the K tiles of a column meet in a 64-bit fixed-point word
        const kx::AwqPlan fp = kx::make_fixed_plan(K, N);
        if (fp.ktiles > 1) {
            rc = kx::resolve_workspace(fp, 1, N, workspace, workspace_bytes, &partials, &counters);
            if (rc != KX_OK) return rc;
#define KX_FARGS x, qweight, scales, qzeros, y, partials, counters, 1, K, N, group_size, fp.coltiles, fp.ktiles, 1, s
            if (fp.rt == 32) kx::launch_awq_gemv<8, 32, 1, kx::kProNone, kx::kEpiStoreFixed>(KX_FARGS);
            else if (fp.waves == 12) kx::launch_awq_gemv<12, 16, 1, kx::kProNone, kx::kEpiStoreFixed>(KX_FARGS);
            else if (fp.waves == 8) kx::launch_awq_gemv<8, 16, 1, kx::kProNone, kx::kEpiStoreFixed>(KX_FARGS);
            else kx::launch_awq_gemv<4, 16, 1, kx::kProNone, kx::kEpiStoreFixed>(KX_FARGS);
#undef KX_FARGS
            return kx::launch_status();
        }
    }
    kx::AwqPlan p = kx::make_plan(M, K, N, group_size, policy);
    rc = kx::resolve_workspace(p, M, N, workspace, workspace_bytes, &partials, &counters);
    if (rc != KX_OK) return rc;
    if (p.mfma) {
        int group_shift = 0;
        while ((1 << group_shift) < group_size) group_shift++;
#define KX_MARGS x, qweight, scales, qzeros, y, partials, counters, M, K, N, group_shift, p.coltiles, p.ktiles, s
#define KX_MFMA_BY_M(KS)                                                        \
    do {                                                                        \
        if (M == 1) kx::launch_awq_gemv_mfma<4, KS, 1, 1>(KX_MARGS);            \
        else if (M == 2) kx::launch_awq_gemv_mfma<4, KS, 2, 1>(KX_MARGS);       \
        else if (M <= 4) kx::launch_awq_gemv_mfma<4, KS, 4, 1>(KX_MARGS);       \
        else if (M <= 8) kx::launch_awq_gemv_mfma<4, KS, 8, 1>(KX_MARGS);       \
        else kx::launch_awq_gemv_mfma<4, KS, 8, 2>(KX_MARGS);                   \
    } while (0)
        if (p.rt == 4) KX_MFMA_BY_M(4);
        else if (p.rt == 2) KX_MFMA_BY_M(2);
        else KX_MFMA_BY_M(1);
#undef KX_MFMA_BY_M
#undef KX_MARGS
        return kx::launch_status();
    }
#define KX_ARGS p, x, qweight, scales, qzeros, y, partials, counters, M, K, N, group_size, s
    if (p.rt == 32) {
        kx::launch_mb<8, 32>(KX_ARGS);
    } else if (p.waves == 12) {  // one activation row by construction of the plan
        kx::launch_awq_gemv<12, 16, 1>(x, qweight, scales, qzeros, y, partials, counters, M, K, N, group_size, p.coltiles,
                                       p.ktiles, p.mtiles, s);
    } else if (p.waves == 8) {
        kx::launch_mb<8, 16>(KX_ARGS);
    } else if (p.rt == 16) {
        kx::launch_mb<4, 16>(KX_ARGS);
    } else {
        kx::launch_mb<4, 8>(KX_ARGS);
    }
#undef KX_ARGS
    return kx::launch_status();
}

extern "C" int kx_gemv_awq_swiglu_bf16(const uint16_t* gate, const uint16_t* up, int32_t act_ld,
                                       const int32_t* qweight, const uint16_t* scales,
                                       const int32_t* qzeros, uint16_t* y, int32_t M, int32_t K,
                                       int32_t N, int32_t group_size, void* workspace,
                                       size_t workspace_bytes, void* stream) {
    if (!gate || !up) return KX_ERR_NULL_POINTER;
    int rc = kx::check_awq_weights(qweight, scales, qzeros, y, M, K, N, group_size);
    if (rc != KX_OK) return rc;
    if (!kx::weights_fit_buffer_loads(K, N)) return KX_ERR_BAD_SHAPE;
    if (act_ld < K) return KX_ERR_BAD_SHAPE;
    if (reinterpret_cast<uintptr_t>(gate) % 2 || reinterpret_cast<uintptr_t>(up) % 2) return KX_ERR_ALIGNMENT;
    kx::FusedInput fi{};
    fi.a = gate;
    fi.b = up;
    fi.ld = act_ld;
    // Several rows go to the matrix cores, as in kx_gemv_awq_bf16, when gate and up can be read 16 bytes at a time
    if (M >= 2 && kx::mfma_shape_ok(N, group_size) && kx::aligned_to(gate, 16) && kx::aligned_to(up, 16) &&
        (act_ld % 8) == 0) {
        const kx::AwqPlan mp = kx::make_mfma_plan(M, K, N, group_size);
        float* partials = nullptr;
        uint32_t* counters = nullptr;
        rc = kx::resolve_workspace(mp, M, N, workspace, workspace_bytes, &partials, &counters);
        if (rc != KX_OK) return rc;
        kx::launch_mfma_fused<kx::kProSwiGLU, kx::kEpiStore>(mp, fi, kx::ResidualTarget{}, nullptr, qweight, scales,
                                                             qzeros, y, partials, counters, M, K, N, group_size,
                                                             kx::as_stream(stream));
        return kx::launch_status();
    }
    const kx::AwqPlan p = kx::make_fused_plan(M, K, N, true);
    float* partials = nullptr;
    uint32_t* counters = nullptr;
    rc = kx::resolve_workspace(p, M, N, workspace, workspace_bytes, &partials, &counters);
    if (rc != KX_OK) return rc;
    kx::launch_fused<kx::kProSwiGLU>(p, fi, qweight, scales, qzeros, y, partials, counters, M, K, N, group_size,
                                     kx::as_stream(stream));
    return kx::launch_status();
}

extern "C" int kx_gemv_awq_addnorm_bf16(const uint16_t* residual, const uint16_t* delta, const uint16_t* gain,
                                        float eps, uint16_t* residual_out, const int32_t* qweight,
                                        const uint16_t* scales, const int32_t* qzeros, uint16_t* y,
                                        int32_t M, int32_t K, int32_t N, int32_t group_size,
                                        void* workspace, size_t workspace_bytes, void* stream) {
    if (!residual || !gain) return KX_ERR_NULL_POINTER;
    int rc = kx::check_awq_weights(qweight, scales, qzeros, y, M, K, N, group_size);
    if (rc != KX_OK) return rc;
    if (!kx::weights_fit_buffer_loads(K, N)) return KX_ERR_BAD_SHAPE;
    if (reinterpret_cast<uintptr_t>(residual) % 16 || reinterpret_cast<uintptr_t>(delta) % 16 ||
        reinterpret_cast<uintptr_t>(gain) % 2 || reinterpret_cast<uintptr_t>(residual_out) % 2) {
        return KX_ERR_ALIGNMENT;
    }
    // every workgroup reads the whole incoming rows while the first column tile writes the outgoing ones
    {
        const size_t row_bytes = static_cast<size_t>(M) * K * sizeof(uint16_t);
        if (kx::ranges_overlap(residual_out, row_bytes, residual, row_bytes) ||
            kx::ranges_overlap(residual_out, row_bytes, delta, row_bytes) ||
            kx::ranges_overlap(residual_out, row_bytes, gain, static_cast<size_t>(K) * sizeof(uint16_t))) {
            return KX_ERR_ALIAS;
        }
    }
    const kx::AwqPlan p = kx::make_fused_plan(M, K, N, false);
    // a thread holds kNormChunks 16-byte pieces of the row for the sum of squares
    if ((K >> 3) > kx::kNormChunks * p.waves * kx::kWave) return KX_ERR_BAD_SHAPE;
    float* partials = nullptr;
    uint32_t* counters = nullptr;
    rc = kx::resolve_workspace(p, M, N, workspace, workspace_bytes, &partials, &counters);
    if (rc != KX_OK) return rc;
    kx::FusedInput fi{};
    fi.a = residual;
    fi.b = delta;
    fi.gain = gain;
    fi.r_out = residual_out;
    fi.ld = K;
    fi.eps = eps;
    if ((K >> 3) <= p.waves * kx::kWave) {
        kx::launch_fused<kx::kProAddNorm>(p, fi, qweight, scales, qzeros, y, partials, counters, M, K, N,
                                          group_size, kx::as_stream(stream));
    } else {
        kx::launch_fused<kx::kProAddNormLong>(p, fi, qweight, scales, qzeros, y, partials, counters, M, K, N,
                                              group_size, kx::as_stream(stream));
    }
    return kx::launch_status();
}

extern "C" int kx_gemv_awq_qkv_rope_bf16(const uint16_t* residual, const uint16_t* delta, const uint16_t* gain,
                                         float eps, uint16_t* residual_out, const int32_t* qweight,
                                         const uint16_t* scales, const int32_t* qzeros, const uint16_t* q_gain,
                                         const uint16_t* k_gain, uint16_t* q_out, uint16_t* k_cache,
                                         uint16_t* v_cache, int32_t n_q_heads, int32_t n_kv_heads,
                                         int32_t head_dim, const int32_t* pos, int32_t cache_positions,
                                         float rope_theta, float qk_eps,
                                         int32_t K, int32_t group_size, void* workspace,
                                         size_t workspace_bytes, void* stream) {
    if (!residual || !gain || !q_gain || !k_gain || !q_out || !k_cache || !v_cache || !pos) {
        return KX_ERR_NULL_POINTER;
    }
    if (head_dim != kx::kHeadDim || n_q_heads < 1 || n_kv_heads < 1 || cache_positions < 1 || !(rope_theta > 1.0f)) {
        return KX_ERR_BAD_SHAPE;
    }
    // a column tile of 256 must hold whole heads
    if ((n_q_heads + 2 * n_kv_heads) % (kx::kTileCols / kx::kHeadDim) != 0) return KX_ERR_BAD_SHAPE;
    const int N = (n_q_heads + 2 * n_kv_heads) * kx::kHeadDim;
    int rc = kx::check_awq_weights(qweight, scales, qzeros, q_out, 1, K, N, group_size);
    if (rc != KX_OK) return rc;
    if (!kx::weights_fit_buffer_loads(K, N)) return KX_ERR_BAD_SHAPE;
    if (reinterpret_cast<uintptr_t>(residual) % 16 || reinterpret_cast<uintptr_t>(delta) % 16 ||
        reinterpret_cast<uintptr_t>(gain) % 2 || reinterpret_cast<uintptr_t>(residual_out) % 2) {
        return KX_ERR_ALIGNMENT;
    }
    {
        const size_t row_bytes = static_cast<size_t>(K) * sizeof(uint16_t);
        if (kx::ranges_overlap(residual_out, row_bytes, residual, row_bytes) ||
            kx::ranges_overlap(residual_out, row_bytes, delta, row_bytes) ||
            kx::ranges_overlap(residual_out, row_bytes, gain, row_bytes)) {
            return KX_ERR_ALIAS;
        }
    }
    const kx::AwqPlan p = kx::make_fused_plan(1, K, N, false);
    if ((K >> 3) > kx::kNormChunks * p.waves * kx::kWave) return KX_ERR_BAD_SHAPE;
    float* partials = nullptr;
    uint32_t* counters = nullptr;
    rc = kx::resolve_workspace(p, 1, N, workspace, workspace_bytes, &partials, &counters);
    if (rc != KX_OK) return rc;
    kx::FusedInput fi{};
    fi.a = residual;
    fi.b = delta;
    fi.gain = gain;
    fi.r_out = residual_out;
    fi.ld = K;
    fi.eps = eps;
    const kx::RopeTarget rope{q_gain, k_gain, q_out, k_cache, v_cache, pos, cache_positions, n_q_heads, n_kv_heads,
                              log2f(rope_theta), qk_eps};
    if ((K >> 3) <= p.waves * kx::kWave) {
        kx::launch_qkv<kx::kProAddNorm>(p, fi, rope, qweight, scales, qzeros, partials, counters, K, N, group_size,
                                        kx::as_stream(stream));
    } else {
        kx::launch_qkv<kx::kProAddNormLong>(p, fi, rope, qweight, scales, qzeros, partials, counters, K, N,
                                            group_size, kx::as_stream(stream));
    }
    return kx::launch_status();
}

extern "C" int kx_gemv_awq_attn_merge_bf16(const void* attn_workspace, size_t attn_workspace_bytes,
                                           int32_t n_q_heads, int32_t n_kv_heads, int32_t head_dim,
                                           int32_t max_positions, const int32_t* qweight, const uint16_t* scales,
                                           const int32_t* qzeros, uint16_t* y, int32_t N, int32_t group_size,
                                           void* workspace, size_t workspace_bytes, void* stream) {
    if (!attn_workspace) return KX_ERR_NULL_POINTER;
    if (head_dim != kx::kHeadDim || n_q_heads < 1 || n_kv_heads < 1 || (n_q_heads % n_kv_heads) != 0 ||
        max_positions < 1) {
        return KX_ERR_BAD_SHAPE;
    }
    const int K = n_q_heads * kx::kHeadDim;
    int rc = kx::check_awq_weights(qweight, scales, qzeros, y, 1, K, N, group_size);
    if (rc != KX_OK) return rc;
    if (!kx::weights_fit_buffer_loads(K, N)) return KX_ERR_BAD_SHAPE;
    const int nchunks = kx::attn_chunks_of(max_positions);
    // a thread holds kMergeHold values of each of its elements: longer contexts take the separate merge
    if (nchunks > kx::kMergeParts * kx::kMergeHold) return KX_ERR_BAD_SHAPE;
    const size_t need = static_cast<size_t>(nchunks) * n_q_heads * (kx::kHeadDim + 2) * sizeof(float);
    if (attn_workspace_bytes < need) return KX_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(attn_workspace) % 16) return KX_ERR_ALIGNMENT;
    kx::AwqPlan p = kx::make_valu_plan(1, K, N, false, false);
    p.mb = 1;
    p.mtiles = 1;
    float* partials = nullptr;
    uint32_t* counters = nullptr;
    rc = kx::resolve_workspace(p, 1, N, workspace, workspace_bytes, &partials, &counters);
    if (rc != KX_OK) return rc;
    kx::FusedInput fi{};
    fi.part_out = static_cast<const float*>(attn_workspace);
    fi.part_ml = fi.part_out + static_cast<size_t>(nchunks) * n_q_heads * kx::kHeadDim;
    fi.nchunks = nchunks;
    fi.heads_per_kv = n_q_heads / n_kv_heads;
    hipStream_t s = kx::as_stream(stream);
#define KX_ARGS nullptr, qweight, scales, qzeros, y, partials, counters, 1, K, N, group_size, p.coltiles, p.ktiles, 1, s, fi
    if (p.waves == 8) kx::launch_awq_gemv<8, 16, 1, kx::kProAttnMerge>(KX_ARGS);
    else kx::launch_awq_gemv<4, 16, 1, kx::kProAttnMerge>(KX_ARGS);  // K = 128: one head
#undef KX_ARGS
    return kx::launch_status();
}

namespace kx {
namespace {

template <int PRO, int EPI>
void launch_chain(const AwqPlan& p, const FusedInput& fi, const RopeTarget& rope, const ResidualTarget& res,
                  const uint16_t* x, const int32_t* qweight, const uint16_t* scales, const int32_t* qzeros,
                  uint16_t* y, float* partials, uint32_t* counters, int K, int N, int group, hipStream_t stream) {
#define KX_ARGS x, qweight, scales, qzeros, y, partials, counters, 1, K, N, group, p.coltiles, p.ktiles, 1, stream, fi, rope, res
    if constexpr (PRO != kProAttnMerge) {
        if (p.rt == 32) {
            launch_awq_gemv<8, 32, 1, PRO, EPI>(KX_ARGS);
            return;
        }
    }
    if constexpr ((PRO == kProNone || PRO == kProSwiGLU) && (EPI == kEpiStore || EPI == kEpiResidual)) {
        if (p.waves == 12) {
            launch_awq_gemv<12, 16, 1, PRO, EPI>(KX_ARGS);
            return;
        }
    }
    if (p.waves == 8) launch_awq_gemv<8, 16, 1, PRO, EPI>(KX_ARGS);
    else if (p.rt == 16) launch_awq_gemv<4, 16, 1, PRO, EPI>(KX_ARGS);
    else if constexpr (PRO != kProAttnMerge) launch_awq_gemv<4, 8, 1, PRO, EPI>(KX_ARGS);
#undef KX_ARGS
}

}  // namespace
}  // namespace kx

extern "C" int kx_gemv_awq_chain_bf16(const kx_chain_desc* d, const int32_t* qweight, const uint16_t* scales,
                                      const int32_t* qzeros, int32_t K, int32_t N, int32_t group_size,
                                      void* workspace, size_t workspace_bytes, void* stream) {
    if (!d) return KX_ERR_NULL_POINTER;
    kx::FusedInput fi{};
    kx::RopeTarget rope{};
    kx::ResidualTarget res{};
    const uint16_t* x = nullptr;
    uint16_t* y = nullptr;
    bool long_rows = true;
    const int rows = d->rows > 0 ? d->rows : 1;
    if (rows > KX_MAX_BATCH || K < 1 || N < 8) return KX_ERR_BAD_SHAPE;
    const int act_ld = d->act_ld > 0 ? d->act_ld : K;
    if (act_ld < K) return KX_ERR_BAD_SHAPE;
    if (rows > 1) {
        // several rows: the matrix-core kernel, which produces activations 16 bytes at a time
        if (d->in_kind == KX_IN_ATTN) return KX_ERR_BAD_SHAPE;
        if (!kx::mfma_shape_ok(N, group_size) || (act_ld % 8) != 0) return KX_ERR_BAD_SHAPE;
    }

    // where the activations come from
    switch (d->in_kind) {
        case KX_IN_ROW:
            if (!d->x) return KX_ERR_NULL_POINTER;
            if (reinterpret_cast<uintptr_t>(d->x) % 16) return KX_ERR_ALIGNMENT;
            x = d->x;
            break;
        case KX_IN_SWIGLU:
            if (!d->gate || !d->up) return KX_ERR_NULL_POINTER;
            if (reinterpret_cast<uintptr_t>(d->gate) % 2 || reinterpret_cast<uintptr_t>(d->up) % 2) return KX_ERR_ALIGNMENT;
            if (rows > 1 && (!kx::aligned_to(d->gate, 16) || !kx::aligned_to(d->up, 16))) return KX_ERR_ALIGNMENT;
            fi.a = d->gate;
            fi.b = d->up;
            fi.ld = act_ld;
            break;
        case KX_IN_ATTN: {
            if (!d->attn_workspace) return KX_ERR_NULL_POINTER;
            if (d->n_q_heads < 1 || d->n_kv_heads < 1 || (d->n_q_heads % d->n_kv_heads) != 0 || d->max_positions < 1 ||
                K != d->n_q_heads * kx::kHeadDim) {
                return KX_ERR_BAD_SHAPE;
            }
            const int nchunks = kx::attn_chunks_of(d->max_positions);
            if (nchunks > kx::kMergeParts * kx::kMergeHold) return KX_ERR_BAD_SHAPE;
            const size_t need = static_cast<size_t>(nchunks) * d->n_q_heads * (kx::kHeadDim + 2) * sizeof(float);
            if (d->attn_workspace_bytes < need) return KX_ERR_WORKSPACE;
            if (reinterpret_cast<uintptr_t>(d->attn_workspace) % 16) return KX_ERR_ALIGNMENT;
            fi.part_out = static_cast<const float*>(d->attn_workspace);
            fi.part_ml = fi.part_out + static_cast<size_t>(nchunks) * d->n_q_heads * kx::kHeadDim;
            fi.nchunks = nchunks;
            fi.heads_per_kv = d->n_q_heads / d->n_kv_heads;
            long_rows = false;  // the merge covers at most 256 rows of K per workgroup
            break;
        }
        case KX_IN_NORM:
            if (!d->norm_row || !d->norm_sumsq || !d->norm_gain) return KX_ERR_NULL_POINTER;
            if (d->norm_parts != (K + kx::kTileCols - 1) / kx::kTileCols || d->norm_parts > kx::kWave) return KX_ERR_BAD_SHAPE;
            if (reinterpret_cast<uintptr_t>(d->norm_row) % 2 || reinterpret_cast<uintptr_t>(d->norm_sumsq) % 16 ||
                reinterpret_cast<uintptr_t>(d->norm_gain) % 2) {
                return KX_ERR_ALIGNMENT;  // the four quarter sums of a tile are read as one 16-byte piece
            }
            if (rows > 1 && (!kx::aligned_to(d->norm_row, 16) || !kx::aligned_to(d->norm_gain, 16))) return KX_ERR_ALIGNMENT;
            fi.a = d->norm_row;
            fi.gain = d->norm_gain;
            fi.eps = d->norm_eps;
            fi.sumsq = d->norm_sumsq;
            fi.sumsq_parts = d->norm_parts;
            fi.ld = act_ld;
            break;
        default: return KX_ERR_BAD_SHAPE;
    }

    // where the result goes
    const uint16_t* out_probe = nullptr;  // any output pointer, for the shared checks
    switch (d->out_kind) {
        case KX_OUT_ROW:
            if (!d->y) return KX_ERR_NULL_POINTER;
            y = d->y;
            out_probe = d->y;
            break;
        case KX_OUT_RESIDUAL:
            if (!d->residual_in || !d->residual_out || !d->sumsq_out) return KX_ERR_NULL_POINTER;
            if (reinterpret_cast<uintptr_t>(d->residual_in) % 2 || reinterpret_cast<uintptr_t>(d->residual_out) % 2 ||
                reinterpret_cast<uintptr_t>(d->sumsq_out) % 4) {
                return KX_ERR_ALIGNMENT;
            }
            {
                // Workgroups of other column tiles still read the activations while the tile that finishes
                // first already writes its 256 columns of the outgoing row: the two must not share a byte.
                // (residual_out may be residual_in itself: a column is read and written by one thread.)
                const size_t out_bytes = static_cast<size_t>(rows) * N * sizeof(uint16_t);
                const size_t in_bytes = (static_cast<size_t>(rows - 1) * act_ld + K) * sizeof(uint16_t);
                if (kx::ranges_overlap(d->residual_out, out_bytes, d->in_kind == KX_IN_NORM ? d->norm_row : nullptr, in_bytes) ||
                    kx::ranges_overlap(d->residual_out, out_bytes, d->in_kind == KX_IN_ROW ? d->x : nullptr, in_bytes) ||
                    kx::ranges_overlap(d->residual_out, out_bytes, d->in_kind == KX_IN_SWIGLU ? d->gate : nullptr, in_bytes) ||
                    kx::ranges_overlap(d->residual_out, out_bytes, d->in_kind == KX_IN_SWIGLU ? d->up : nullptr, in_bytes)) {
                    return KX_ERR_ALIAS;
                }
                if (d->residual_out != d->residual_in &&
                    kx::ranges_overlap(d->residual_out, out_bytes, d->residual_in, out_bytes)) {
                    return KX_ERR_ALIAS;  // a shifted overlap: another thread's column would be overwritten
                }
            }
            res.in = d->residual_in;
            res.out = d->residual_out;
            res.sumsq = d->sumsq_out;
            out_probe = d->residual_out;
            break;
        case KX_OUT_QKV_ROPE:
            if (!d->q_gain || !d->k_gain || !d->q_out || !d->k_cache || !d->v_cache || !d->pos) return KX_ERR_NULL_POINTER;
            if (d->rope_n_q_heads < 1 || d->rope_n_kv_heads < 1 || d->cache_positions < 1 || !(d->rope_theta > 1.0f) ||
                N != (d->rope_n_q_heads + 2 * d->rope_n_kv_heads) * kx::kHeadDim ||
                (d->rope_n_q_heads + 2 * d->rope_n_kv_heads) % (kx::kTileCols / kx::kHeadDim) != 0) {
                return KX_ERR_BAD_SHAPE;
            }
            // several rows are several sequences, each with a cache pair of its own
            if (rows > 1 && d->cache_stride < static_cast<size_t>(d->cache_positions) * d->rope_n_kv_heads * kx::kHeadDim) {
                return KX_ERR_BAD_SHAPE;
            }
            rope = kx::RopeTarget{d->q_gain, d->k_gain, d->q_out, d->k_cache, d->v_cache, d->pos, d->cache_positions,
                                  d->rope_n_q_heads, d->rope_n_kv_heads, log2f(d->rope_theta), d->qk_eps};
            out_probe = d->q_out;
            break;
        default: return KX_ERR_BAD_SHAPE;
    }
    // 8-byte alignment is what the plain store asks of y; the other outputs are written per element
    int rc = kx::check_awq_weights(qweight, scales, qzeros, out_probe, rows, K, N, group_size, d->out_kind == KX_OUT_ROW);
    if (rc != KX_OK) return rc;
    if (d->in_kind != KX_IN_ROW && !kx::weights_fit_buffer_loads(K, N)) return KX_ERR_BAD_SHAPE;
    if (d->in_kind == KX_IN_ATTN && (K % kx::kHeadDim) != 0) return KX_ERR_BAD_SHAPE;

    if (rows > 1) {
        const kx::AwqPlan mp = kx::make_mfma_plan(rows, K, N, group_size);
        float* partials = nullptr;
        uint32_t* counters = nullptr;
        rc = kx::resolve_workspace(mp, rows, N, workspace, workspace_bytes, &partials, &counters);
        if (rc != KX_OK) return rc;
        hipStream_t s = kx::as_stream(stream);
#define KX_MCHAIN(PRO, EPI) kx::launch_mfma_fused<PRO, EPI>(mp, fi, res, x, qweight, scales, qzeros, y, partials, counters, rows, K, N, group_size, s, rope, d->cache_stride)
#define KX_MBY_OUT(PRO)                                                               \
    do {                                                                              \
        if (d->out_kind == KX_OUT_ROW) KX_MCHAIN(PRO, kx::kEpiStore);                 \
        else if (d->out_kind == KX_OUT_RESIDUAL) KX_MCHAIN(PRO, kx::kEpiResidual);    \
        else KX_MCHAIN(PRO, kx::kEpiQkRope);                                          \
    } while (0)
        switch (d->in_kind) {
            case KX_IN_ROW: KX_MBY_OUT(kx::kProNone); break;
            case KX_IN_SWIGLU: KX_MBY_OUT(kx::kProSwiGLU); break;
            default: KX_MBY_OUT(kx::kProPreNorm); break;
        }
#undef KX_MBY_OUT
#undef KX_MCHAIN
        return kx::launch_status();
    }

    const bool plain_ends = (d->in_kind == KX_IN_ROW || d->in_kind == KX_IN_SWIGLU) &&
                            (d->out_kind == KX_OUT_ROW || d->out_kind == KX_OUT_RESIDUAL);
    kx::AwqPlan p = kx::make_valu_plan(1, K, N, long_rows, plain_ends);
    p.mb = 1;
    p.mtiles = 1;
    float* partials = nullptr;
    uint32_t* counters = nullptr;
    rc = kx::resolve_workspace(p, 1, N, workspace, workspace_bytes, &partials, &counters);
    if (rc != KX_OK) return rc;
    hipStream_t s = kx::as_stream(stream);

#define KX_CHAIN(PRO, EPI) kx::launch_chain<PRO, EPI>(p, fi, rope, res, x, qweight, scales, qzeros, y, partials, counters, K, N, group_size, s)
#define KX_BY_OUT(PRO)                                                                   \
    do {                                                                                 \
        if (d->out_kind == KX_OUT_ROW) KX_CHAIN(PRO, kx::kEpiStore);                     \
        else if (d->out_kind == KX_OUT_RESIDUAL) KX_CHAIN(PRO, kx::kEpiResidual);        \
        else KX_CHAIN(PRO, kx::kEpiQkRope);                                              \
    } while (0)
    switch (d->in_kind) {
        case KX_IN_ROW: KX_BY_OUT(kx::kProNone); break;
        case KX_IN_SWIGLU: KX_BY_OUT(kx::kProSwiGLU); break;
        case KX_IN_ATTN: KX_BY_OUT(kx::kProAttnMerge); break;
        default: KX_BY_OUT(kx::kProPreNorm); break;
    }
#undef KX_BY_OUT
#undef KX_CHAIN
    return kx::launch_status();
}
