// Fused INT4 AWQ dequantise + GEMV for gfx950 (wave64), M <= 16.
//
//   y[m,n] = sum_k x[m,k] * (q[k,n] - z[k/G,n]) * s[k/G,n]
//
// The packed stream is consumed as it lies in memory: qweight int32 [K, N/8], one word = eight
// columns of one row.  A lane owns one word column and RT consecutive rows (all inside one
// quantisation group), so that scale and zero point are applied once per lane and column:
//
//   y_part[n] = s[g,n] * ( sum_r q[k0+r,n] * x[k0+r]  -  z[g,n] * sum_r x[k0+r] )
//
// A wave covers WC consecutive word columns (WC*4 bytes of each row, contiguous) times 64/WC row
// slots; a workgroup stacks WAVES waves along K.  Partial sums meet in LDS, then across
// workgroups in a caller-provided workspace: the last workgroup to arrive at a column tile adds
// the partials in a fixed order, which keeps the result bitwise reproducible.
#include "kx_common.h"

#include <stdlib.h>

namespace kx {
namespace {

struct AwqPlan {
    int waves;     // waves per workgroup (4, 8 or 16)
    int mb;        // activation rows handled per workgroup (1, 2, 4 or 8)
    int coltiles;  // tiles of WC word columns
    int ktiles;    // workgroups along K
    int mtiles;    // ceil(M / mb)
};

constexpr int kWC = 32;  // word columns per wave: 128 contiguous bytes of a row, 256 output columns
constexpr int kRT = 8;   // consecutive rows per lane

inline int rows_per_block(int waves) {
    return waves * (kWave / kWC) * kRT;
}

inline AwqPlan make_plan(int M, int K, int N) {
    AwqPlan p;
    p.mb = M >= 8 ? 8 : (M >= 4 ? 4 : (M >= 2 ? 2 : 1));
    p.mtiles = (M + p.mb - 1) / p.mb;
    int nw = N / 8;
    p.coltiles = (nw + kWC - 1) / kWC;
    p.waves = 16;
    static const int forced = [] {
        const char* e = getenv("KX_AWQ_WAVES");
        return e ? atoi(e) : 0;
    }();
    if (forced == 4 || forced == 8 || forced == 16) {
        p.waves = forced;
    } else {
        // Stack as much of K as possible inside one workgroup (fewer partial sums to exchange),
        // but keep at least one workgroup per compute unit.
        while (p.waves > 4 &&
               static_cast<long>(p.coltiles) * ((K + rows_per_block(p.waves) - 1) / rows_per_block(p.waves)) < 256) {
            p.waves /= 2;
        }
    }
    int kb = rows_per_block(p.waves);
    p.ktiles = (K + kb - 1) / kb;
    return p;
}

// Device-scope (all XCDs) write-through store and cache-bypassing load for the split-K exchange.
__device__ __forceinline__ void store_agent(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_agent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Columns held by the bytes of (w & 0x0F0F0F0F) and ((w >> 4) & 0x0F0F0F0F):
// byte b of the low mask is nibble 2b -> column order_of(2b); of the high mask nibble 2b+1.
template <int MB>
__device__ __forceinline__ void accumulate_word(uint32_t w, const float (&xv)[MB], float (&acc)[MB][8]) {
    uint32_t lo = w & 0x0F0F0F0Fu;
    uint32_t hi = (w >> 4) & 0x0F0F0F0Fu;
    float q[8];
    q[order_of(0)] = static_cast<float>(lo & 0xffu);
    q[order_of(2)] = static_cast<float>((lo >> 8) & 0xffu);
    q[order_of(4)] = static_cast<float>((lo >> 16) & 0xffu);
    q[order_of(6)] = static_cast<float>(lo >> 24);
    q[order_of(1)] = static_cast<float>(hi & 0xffu);
    q[order_of(3)] = static_cast<float>((hi >> 8) & 0xffu);
    q[order_of(5)] = static_cast<float>((hi >> 16) & 0xffu);
    q[order_of(7)] = static_cast<float>(hi >> 24);
#pragma unroll
    for (int m = 0; m < MB; m++) {
#pragma unroll
        for (int c = 0; c < 8; c++) {
            acc[m][c] = __builtin_fmaf(q[c], xv[m], acc[m][c]);
        }
    }
}

template <int WAVES, int MB>
__global__ __launch_bounds__(WAVES * kWave) void awq_gemv_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    uint16_t* __restrict__ y, float* __restrict__ partials, uint32_t* __restrict__ counters,
    int M, int K, int N, int group, int coltiles, int ktiles) {
    constexpr int SLOTS_PER_WAVE = kWave / kWC;
    constexpr int SLOTS = WAVES * SLOTS_PER_WAVE;
    constexpr int KB = SLOTS * kRT;
    constexpr int TILE_COLS = kWC * 8;
    constexpr int THREADS = WAVES * kWave;

    __shared__ float red[SLOTS][TILE_COLS];
    __shared__ int s_last;

    const int tid = threadIdx.x;
    const int ct = blockIdx.x % coltiles;
    const int kt = blockIdx.x / coltiles;
    const int m0 = blockIdx.y * MB;
    const int nw = N >> 3;

    const int wc = tid % kWC;           // word column inside the tile
    const int slot = tid / kWC;         // row slot inside the workgroup
    const int wcg = ct * kWC + wc;      // word column in the matrix
    const int k0 = kt * KB + slot * kRT;
    const bool active = (wcg < nw) && (k0 < K);

    float acc[MB][8];
#pragma unroll
    for (int m = 0; m < MB; m++) {
#pragma unroll
        for (int c = 0; c < 8; c++) acc[m][c] = 0.0f;
    }

    if (active) {
        // Issue every weight load of this lane before anything consumes them.
        uint32_t w[kRT];
        const uint32_t* wp = qweight + static_cast<size_t>(k0) * nw + wcg;
#pragma unroll
        for (int r = 0; r < kRT; r++) {
            w[r] = __builtin_nontemporal_load(wp + static_cast<size_t>(r) * nw);
        }
        const int g = k0 / group;
        const uint32_t zw = qzeros[static_cast<size_t>(g) * nw + wcg];
        const uint4 sraw = *reinterpret_cast<const uint4*>(scales + static_cast<size_t>(g) * N + 8 * wcg);

        float xs[MB][kRT];
        float xsum[MB];
#pragma unroll
        for (int m = 0; m < MB; m++) {
            xsum[m] = 0.0f;
            if (m0 + m < M) {
                const uint4 xr = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(m0 + m) * K + k0);
                const uint32_t xw[4] = {xr.x, xr.y, xr.z, xr.w};
#pragma unroll
                for (int r = 0; r < kRT; r++) {
                    uint32_t bits = (r & 1) ? (xw[r >> 1] & 0xffff0000u) : (xw[r >> 1] << 16);
                    xs[m][r] = __uint_as_float(bits);
                    xsum[m] += xs[m][r];
                }
            } else {
#pragma unroll
                for (int r = 0; r < kRT; r++) xs[m][r] = 0.0f;
            }
        }

#pragma unroll
        for (int r = 0; r < kRT; r++) {
            float xv[MB];
#pragma unroll
            for (int m = 0; m < MB; m++) xv[m] = xs[m][r];
            accumulate_word<MB>(w[r], xv, acc);
        }

        // zero point and scale, once per lane and column
        const uint32_t zlo = zw & 0x0F0F0F0Fu;
        const uint32_t zhi = (zw >> 4) & 0x0F0F0F0Fu;
        float z[8];
        z[order_of(0)] = static_cast<float>(zlo & 0xffu);
        z[order_of(2)] = static_cast<float>((zlo >> 8) & 0xffu);
        z[order_of(4)] = static_cast<float>((zlo >> 16) & 0xffu);
        z[order_of(6)] = static_cast<float>(zlo >> 24);
        z[order_of(1)] = static_cast<float>(zhi & 0xffu);
        z[order_of(3)] = static_cast<float>((zhi >> 8) & 0xffu);
        z[order_of(5)] = static_cast<float>((zhi >> 16) & 0xffu);
        z[order_of(7)] = static_cast<float>(zhi >> 24);
        const uint32_t sw[4] = {sraw.x, sraw.y, sraw.z, sraw.w};
        float s[8];
#pragma unroll
        for (int c = 0; c < 8; c++) {
            s[c] = f16_bits_to_f32(static_cast<uint16_t>((c & 1) ? (sw[c >> 1] >> 16) : (sw[c >> 1] & 0xffffu)));
        }
#pragma unroll
        for (int m = 0; m < MB; m++) {
#pragma unroll
            for (int c = 0; c < 8; c++) {
                acc[m][c] = s[c] * __builtin_fmaf(-z[c], xsum[m], acc[m][c]);
            }
        }
    }

    // Reduce the row slots of the workgroup through LDS, one activation row at a time.
    const int col = ct * TILE_COLS + tid;  // column owned by thread tid < TILE_COLS afterwards
    for (int m = 0; m < MB; m++) {
        float4* dst = reinterpret_cast<float4*>(&red[slot][8 * wc]);
        dst[0] = make_float4(acc[m][0], acc[m][1], acc[m][2], acc[m][3]);
        dst[1] = make_float4(acc[m][4], acc[m][5], acc[m][6], acc[m][7]);
        __syncthreads();
        if (tid < TILE_COLS) {
            float sum = 0.0f;
#pragma unroll
            for (int sl = 0; sl < SLOTS; sl++) sum += red[sl][tid];
            if (col < N && m0 + m < M) {
                if (ktiles == 1) {
                    y[static_cast<size_t>(m0 + m) * N + col] = f32_to_bf16(sum);
                } else {
                    store_agent(&partials[(static_cast<size_t>(kt) * M + (m0 + m)) * N + col], sum);
                }
            }
        }
        __syncthreads();
    }
    if (ktiles == 1) return;

    // Arrival counter per (column tile, activation tile); the last workgroup finishes the sum.
    // The partials were stored write-through at device scope, so it is enough that every wave
    // has seen its stores acknowledged before the counter moves: a workgroup-scope release
    // (a wait, no cache-wide write-back) followed by the barrier gives exactly that.  A
    // device-scope fence here would write back and invalidate the whole L2 once per workgroup.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    const int cidx = blockIdx.y * coltiles + ct;
    if (tid == 0) {
        uint32_t prev = __hip_atomic_fetch_add(&counters[cidx], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (prev == static_cast<uint32_t>(ktiles - 1));
    }
    __syncthreads();
    if (!s_last) return;
    if (tid < TILE_COLS && col < N) {
        for (int m = 0; m < MB && m0 + m < M; m++) {
            float sum = 0.0f;
            const float* pp = partials + static_cast<size_t>(m0 + m) * N + col;
            for (int t = 0; t < ktiles; t++) {
                sum += load_agent(pp + static_cast<size_t>(t) * M * N);
            }
            y[static_cast<size_t>(m0 + m) * N + col] = f32_to_bf16(sum);
        }
    }
    if (tid == 0) {
        // leave the workspace ready for the next launch
        __hip_atomic_store(&counters[cidx], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    (void)THREADS;
}

template <int WAVES, int MB>
void launch(const AwqPlan& p, const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
            const int32_t* qzeros, uint16_t* y, float* partials, uint32_t* counters, int M, int K,
            int N, int group, hipStream_t stream) {
    dim3 grid(p.coltiles * p.ktiles, p.mtiles, 1);
    dim3 block(WAVES * kWave, 1, 1);
    hipLaunchKernelGGL((awq_gemv_kernel<WAVES, MB>), grid, block, 0, stream, x,
                       reinterpret_cast<const uint32_t*>(qweight), scales,
                       reinterpret_cast<const uint32_t*>(qzeros), y, partials, counters, M, K, N,
                       group, p.coltiles, p.ktiles);
}

template <int WAVES>
void launch_mb(const AwqPlan& p, const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
               const int32_t* qzeros, uint16_t* y, float* partials, uint32_t* counters, int M,
               int K, int N, int group, hipStream_t stream) {
    switch (p.mb) {
        case 1: launch<WAVES, 1>(p, x, qweight, scales, qzeros, y, partials, counters, M, K, N, group, stream); break;
        case 2: launch<WAVES, 2>(p, x, qweight, scales, qzeros, y, partials, counters, M, K, N, group, stream); break;
        case 4: launch<WAVES, 4>(p, x, qweight, scales, qzeros, y, partials, counters, M, K, N, group, stream); break;
        default: launch<WAVES, 8>(p, x, qweight, scales, qzeros, y, partials, counters, M, K, N, group, stream); break;
    }
}

__global__ void fill_zero_u32(uint32_t* p, size_t n) {
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

}  // namespace
}  // namespace kx

extern "C" size_t kx_gemv_workspace_bytes(int32_t M, int32_t K, int32_t N) {
    if (M < 1 || M > KX_MAX_BATCH || K < 1 || N < 8) return 0;
    // Upper bound over every plan: the smallest workgroup stacks 4 waves along K.
    size_t kb = static_cast<size_t>(kx::rows_per_block(4));
    size_t ktiles = (static_cast<size_t>(K) + kb - 1) / kb;
    return kx::kCounterBytes + ktiles * static_cast<size_t>(M) * static_cast<size_t>(N) * sizeof(float);
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
        reinterpret_cast<uintptr_t>(y) % 2) {
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
    switch (p.waves) {
        case 4: kx::launch_mb<4>(p, x, qweight, scales, qzeros, y, partials, counters, M, K, N, group_size, s); break;
        case 8: kx::launch_mb<8>(p, x, qweight, scales, qzeros, y, partials, counters, M, K, N, group_size, s); break;
        default: kx::launch_mb<16>(p, x, qweight, scales, qzeros, y, partials, counters, M, K, N, group_size, s); break;
    }
    return kx::launch_status();
}
