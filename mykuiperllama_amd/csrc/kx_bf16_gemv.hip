// BF16 GEMV fallback for gfx950: y[m,n] = sum_k x[m,k] * W[n,k], W bf16 row-major [N, K].
//
// One or two activation rows: one wave per output row, the 64 lanes walk the row in 16-byte pieces
// (eight bf16 each), pairs along K go through the packed bf16 dot instruction with an fp32
// accumulator, and the lanes meet in a wave-wide sum at the end.  Rows are contiguous, so every load
// is a full 1 KiB per wave.  Three to sixteen rows: matrix cores, sixteen output rows per workgroup
// (second kernel below).
#include "kx_common.h"

namespace kx {
namespace {

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
    bf16x2 va, vb;
    __builtin_memcpy(&va, &a, 4);
    __builtin_memcpy(&vb, &b, 4);
    return __builtin_amdgcn_fdot2_f32_bf16(va, vb, c, false);
}

constexpr int kRowsPerBlock = 4;  // one wave each
// 16-byte weight loads in flight per lane: a row of 4096 in one sweep (four measured slower for
// every M, also where several activation rows compete for the registers)
constexpr int kUnroll = 8;

template <int MB>
__global__ __launch_bounds__(kRowsPerBlock * kWave) void bf16_gemv_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, uint16_t* __restrict__ y,
    int M, int K, int N, int m0) {
    const int lane = threadIdx.x % kWave;
    const int n = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
    // A wave past the last row works on the last row again and stores nothing: no wave leaves
    // early, no load sits under a condition.
    const int n_ld = n < N ? n : N - 1;
    const int chunks = K >> 3;  // 16-byte pieces per row
    const u32x4* wrow = reinterpret_cast<const u32x4*>(w + static_cast<size_t>(n_ld) * K);
    const uint4* xrow[MB];
#pragma unroll
    for (int m = 0; m < MB; m++) {
        const int mr = m0 + m < M ? m0 + m : M - 1;  // rows past M repeat the last one, never stored
        xrow[m] = reinterpret_cast<const uint4*>(x + static_cast<size_t>(mr) * K);
    }

    float acc[MB];
#pragma unroll
    for (int m = 0; m < MB; m++) acc[m] = 0.0f;

    // Full sweeps of kUnroll pieces per lane, then the rest of the row two pieces per lane at a time
    // (K = 5120: one full sweep and one short one).  Inside a sweep the loads are straight-line code
    // and all in flight together; a load under a condition becomes a branch with a full wait behind it.
    auto consume = [&](const u32x4& wv, int c, bool live) {
        const uint32_t w0 = live ? wv.x : 0u, w1 = live ? wv.y : 0u;
        const uint32_t w2 = live ? wv.z : 0u, w3 = live ? wv.w : 0u;
#pragma unroll
        for (int m = 0; m < MB; m++) {
            const uint4 xv = xrow[m][c];
            acc[m] = dot2_bf16(w0, xv.x, acc[m]);
            acc[m] = dot2_bf16(w1, xv.y, acc[m]);
            acc[m] = dot2_bf16(w2, xv.z, acc[m]);
            acc[m] = dot2_bf16(w3, xv.w, acc[m]);
        }
    };
    int base = 0;  // first piece of the sweep, the same in every lane
    for (; base + kWave * kUnroll <= chunks; base += kWave * kUnroll) {
        u32x4 wv[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) wv[u] = __builtin_nontemporal_load(wrow + base + lane + u * kWave);
        __builtin_amdgcn_sched_barrier(0);  // every weight load is out before the first is waited for
#pragma unroll
        for (int u = 0; u < kUnroll; u++) consume(wv[u], base + lane + u * kWave, true);
    }
    constexpr int kTail = 2;
    for (; base < chunks; base += kWave * kTail) {
        // clamped addresses, masked weights
        u32x4 wv[kTail];
#pragma unroll
        for (int u = 0; u < kTail; u++) {
            const int c = base + lane + u * kWave;
            wv[u] = __builtin_nontemporal_load(wrow + (c < chunks ? c : chunks - 1));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < kTail; u++) {
            const int c = base + lane + u * kWave;
            consume(wv[u], c < chunks ? c : chunks - 1, c < chunks);
        }
    }
#pragma unroll
    for (int m = 0; m < MB; m++) acc[m] = wave_sum(acc[m]);
    if (lane == 0 && n < N) {
#pragma unroll
        for (int m = 0; m < MB; m++) {
            // a plain store: one wave owns one column, and two-byte write-through stores from 150 000 waves cost
            // the lm_head launch 8 us
            if (m0 + m < M) y[static_cast<size_t>(m0 + m) * N + n] = f32_to_bf16(acc[m]);
        }
    }
}

// Three to sixteen activation rows: matrix cores, one pass over W whatever M is.
// v_mfma_f32_16x16x32_bf16 with A = the activations (row m = lane % 16, zero rows past M) and
// B = sixteen rows of W (column n = lane % 16): lane (c, b) supplies x[c][32 s + 8 b .. + 7] and
// W[n0 + c][32 s + 8 b .. + 7], sixteen contiguous bytes each, and receives y[4 b + v][n0 + c].
// A workgroup owns BLOCKS blocks of sixteen output columns, which share every A operand.  One block
// with eight steps in flight serves up to eight rows (lm_head 151936 x 4096: 270 us at M = 3..5, 300 at
// 8); from nine rows on four blocks with four steps in flight each, so that the activation rows come out
// of L2 once per 64 columns instead of once per 16 - at sixteen rows they are as many bytes as the sixteen
// rows of W they meet, and with one block the L2 traffic for x equalled the HBM traffic for W (370 us at
// M = 16, 299 with four blocks; at M = 3 four blocks are the slower choice, 297 us).  Its four waves take the
// 32-element steps of K in turn (step s goes to wave s % 4; runs of consecutive steps per wave measured
// slower) in sweeps of UNROLL steps with all loads of a sweep in flight together, and meet in LDS.  Addresses are clamped, what lies past K or M is zeroed
// in both operands; per output the additions run in the same order whatever kMfmaBlocks is.
constexpr int kMfmaWaves = 4;

template <int kMfmaBlocks, int kMfmaUnroll>
__global__ __launch_bounds__(kMfmaWaves * kWave) void bf16_gemv_mfma_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, uint16_t* __restrict__ y, int M, int K, int N) {
    __shared__ float red[kMfmaWaves][kMfmaBlocks][4][kWave];
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int c = lane % 16;
    const int b = lane / 16;
    const int n0 = blockIdx.x * 16 * kMfmaBlocks;
    const int m_ld = c < M ? c : M - 1;
    const uint16_t* wrow[kMfmaBlocks];
#pragma unroll
    for (int j = 0; j < kMfmaBlocks; j++) {
        const int n = n0 + 16 * j + c;
        wrow[j] = w + static_cast<size_t>(n < N ? n : N - 1) * K;
    }
    const uint16_t* xrow = x + static_cast<size_t>(m_ld) * K;
    const bool row_live = c < M;
    const int k_last = K - 8;  // K is a multiple of eight

    f32x4v acc[kMfmaBlocks];
#pragma unroll
    for (int j = 0; j < kMfmaBlocks; j++) acc[j] = f32x4v{0.0f, 0.0f, 0.0f, 0.0f};
    constexpr int kSweep = 32 * kMfmaWaves * kMfmaUnroll;  // elements of K a workgroup covers per sweep
    for (int k0 = 32 * wave; k0 < K; k0 += kSweep) {
        u32x4 wv[kMfmaUnroll][kMfmaBlocks], xv[kMfmaUnroll];
#pragma unroll
        for (int u = 0; u < kMfmaUnroll; u++) {
            const int k = k0 + 32 * kMfmaWaves * u + 8 * b;
            xv[u] = *reinterpret_cast<const u32x4*>(xrow + (k < K ? k : k_last));
        }
#pragma unroll
        for (int u = 0; u < kMfmaUnroll; u++) {
            const int k = k0 + 32 * kMfmaWaves * u + 8 * b;
#pragma unroll
            for (int j = 0; j < kMfmaBlocks; j++) {
                wv[u][j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[j] + (k < K ? k : k_last)));
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // every load of the sweep is out before the first is waited for
#pragma unroll
        for (int u = 0; u < kMfmaUnroll; u++) {
            const bool live = k0 + 32 * kMfmaWaves * u + 8 * b < K;
            const bool a_live = live && row_live;
            const bf16x8 a_op = as_bf16x8(a_live ? xv[u].x : 0u, a_live ? xv[u].y : 0u, a_live ? xv[u].z : 0u,
                                          a_live ? xv[u].w : 0u);
#pragma unroll
            for (int j = 0; j < kMfmaBlocks; j++) {
                const bf16x8 b_op = as_bf16x8(live ? wv[u][j].x : 0u, live ? wv[u][j].y : 0u, live ? wv[u][j].z : 0u,
                                              live ? wv[u][j].w : 0u);
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_op, b_op, acc[j], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < kMfmaBlocks; j++) {
#pragma unroll
        for (int v = 0; v < 4; v++) red[wave][j][v][lane] = acc[j][v];
    }
    __syncthreads();
    // wave j finishes block j
    static_assert(kMfmaBlocks <= kMfmaWaves, "one wave per block of sixteen columns in the final sum");
    const int n = n0 + 16 * wave + c;
    if (wave < kMfmaBlocks && n < N) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int m = 4 * b + v;
            const float sum = (red[0][wave][v][lane] + red[1][wave][v][lane]) + (red[2][wave][v][lane] + red[3][wave][v][lane]);
            if (m < M) y[static_cast<size_t>(m) * N + n] = f32_to_bf16(sum);
        }
    }
}

}  // namespace
}  // namespace kx

extern "C" int kx_gemv_bf16(const uint16_t* x, const uint16_t* w, uint16_t* y, int32_t M, int32_t K,
                            int32_t N, void* workspace, size_t workspace_bytes, void* stream) {
    (void)workspace;
    (void)workspace_bytes;
    if (!x || !w || !y) return KX_ERR_NULL_POINTER;
    if (M < 1 || M > KX_MAX_BATCH || K < 8 || (K % 8) != 0 || N < 1) return KX_ERR_BAD_SHAPE;
    if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(w) % 16 ||
        reinterpret_cast<uintptr_t>(y) % 2) {
        return KX_ERR_ALIGNMENT;
    }
    hipStream_t s = kx::as_stream(stream);
    if (M >= 3) {
        // One pass on the matrix cores; the vector kernel, whose every wave reads the activation rows for
        // itself, needs 310 us on lm_head 151936 x 4096 for four rows and a pass over W per four rows beyond that.
        if (M <= 8) {
            hipLaunchKernelGGL((kx::bf16_gemv_mfma_kernel<1, 8>), dim3((N + 15) / 16), dim3(kx::kMfmaWaves * kx::kWave), 0,
                               s, x, w, y, M, K, N);
        } else {
            hipLaunchKernelGGL((kx::bf16_gemv_mfma_kernel<4, 4>), dim3((N + 63) / 64), dim3(kx::kMfmaWaves * kx::kWave), 0,
                               s, x, w, y, M, K, N);
        }
        return kx::launch_status();
    }
    const dim3 grid((N + kx::kRowsPerBlock - 1) / kx::kRowsPerBlock);
    const dim3 block(kx::kRowsPerBlock * kx::kWave);
    if (M == 1) {
        hipLaunchKernelGGL((kx::bf16_gemv_kernel<1>), grid, block, 0, s, x, w, y, M, K, N, 0);
    } else {
        hipLaunchKernelGGL((kx::bf16_gemv_kernel<2>), grid, block, 0, s, x, w, y, M, K, N, 0);
    }
    return kx::launch_status();
}
