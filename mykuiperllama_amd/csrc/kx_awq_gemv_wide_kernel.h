// A measured alternative to the one-shot MFMA kernel, kept selectable (KX_POLICY_WIDE of the internal entry
// point) so that the comparison can be repeated: 16-byte, workgroup-cooperative loads through LDS.
//
//   y[m,n] = sum_k x[m,k] * (q[k,n] - z[k/G,n]) * s[k/G,n]          (gfx950, v_mfma_f32_16x16x32_bf16, M <= 16)
//
// Arithmetic and reduction are those of kx_awq_gemv_mfma_kernel.h.  What differs is how the operands reach the
// lanes.  A compute unit of this machine takes one vector-memory instruction of a wave about every 12 ns
// whatever its width (measured on loads that hit L1: 4, 8 and 16 bytes per lane alike), so fewer, wider
// instructions get a workgroup's requests out sooner.  Here every thread fetches its share of the workgroup's
// tile (KB rows of K x 128 bytes, 256 output columns) with 16-byte loads - a wave instruction is eight rows x
// 128 contiguous bytes - and the tile passes through LDS, from which each wave reads its 32-row steps back in
// the layout the MFMA B operand wants (lane (c, b): rows 8b..8b+7 of word pair c).  Scales and zero words of the
// quantisation groups the tile touches and the activation rows are staged in LDS the same way.  Per 4 KiB of
// packed weights a workgroup issues about 4.5 vector-memory instructions against 13 in the one-shot MFMA
// kernel and 20 in the vector kernel.
//
// What it measured (us per launch, M = 1, cold weights, this kernel / one-shot MFMA kernel): 4096->1024 5.5 / 5.1,
// 4096->4096 6.6 / 5.8, 4096->12288 10.2 / 8.5, 4096->24576 16.1 / 13.0, 5120->51200 34.8 / 29.3: slower
// everywhere.  The load phase of the one-shot kernels is not what holds them back (with the arithmetic and
// the exchange compiled out they run within 0.1-0.5 us of a kernel that only reads the same bytes); what the
// detour through LDS adds - a workgroup-wide barrier between the last byte's arrival and the first product, and
// 64 KiB of LDS traffic per workgroup - is more than the issue slots it saves.  The one-shot kernels stay the
// default.
#ifndef KX_AWQ_GEMV_WIDE_KERNEL_H
#define KX_AWQ_GEMV_WIDE_KERNEL_H

#include "kx_awq_gemv_mfma_kernel.h"
#include "kx_common.h"
#include "kx_splitk_exchange.h"

namespace kx {

constexpr int kWideWaves = 4;
constexpr int kWideThreads = kWideWaves * kWave;

// KS: 32-row steps per wave (the wave's rows lie in one quantisation group);
// MC: activation rows per LDS round of the final reduction; ROUNDS: 2 for M > 8, else 1.
template <int KS, int MC, int ROUNDS>
__global__ __launch_bounds__(kWideThreads, 2) void awq_gemv_wide_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    uint16_t* __restrict__ y, float* __restrict__ partials, uint32_t* __restrict__ counters,
    int M, int K, int N, int group_shift, int ktiles) {
    constexpr int WAVES = kWideWaves;
    constexpr int WROWS = KS * kStepRows;  // rows of K per wave
    constexpr int KB = WAVES * WROWS;      // rows of K per workgroup
    constexpr int ROWS = MC * ROUNDS;      // activation rows this kernel carries (>= M)
    constexpr int LOADS = KB / 32;         // 16-byte weight loads per thread: 32 rows x 128 B per round
    constexpr int XPITCH = KB + 8;         // bf16 elements between staged activation rows (16 bytes of padding)
    constexpr int XPIECES = ROWS * (KB / 8);  // 16-byte pieces of the staged activations
    constexpr int XPASSES = (XPIECES + kWideThreads - 1) / kWideThreads;
    static_assert(WAVES * kWave == kTileCols, "one thread per tile column");

    // The tile of packed weights and, once it has been consumed, the waves' sums share one block of LDS.
    constexpr int TILE_BYTES = KB * 128;
    constexpr int RED_BYTES = WAVES * MC * kTileCols * 4;
    constexpr int BLOCK_BYTES = TILE_BYTES > RED_BYTES ? TILE_BYTES : RED_BYTES;
    __shared__ __attribute__((aligned(16))) unsigned char s_block[BLOCK_BYTES];
    __shared__ __attribute__((aligned(16))) uint16_t s_x[ROWS][XPITCH];
    __shared__ __attribute__((aligned(16))) uint16_t s_sc[WAVES][kTileCols];  // scales of each wave's group
    __shared__ __attribute__((aligned(16))) uint32_t s_zw[WAVES][kTileCols / 8];
    __shared__ float xs_red[WAVES][MC];
    __shared__ uint32_t s_prev;

    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int lane = tid % kWave;
    const int c = lane % 16;  // word pair c of the tile, MFMA column c
    const int b = lane / 16;  // k block inside a step, D row block
    const int ct = blockIdx.x;
    const int kt = blockIdx.y;
    const int nw = N >> 3;
    const int k_base = kt * KB;

    // ---- loads, all issued before anything is consumed; every address is clamped into its tensor ----
    // weights: round i brings rows k_base + 32 i .. + 31, thread t the 16 bytes (t % 8) of row t / 8
    u32x4 wld[LOADS];
    {
        const int wcol = ct * 32 + (tid & 7) * 4;
        const int wcol_c = wcol < nw ? wcol : nw - 4;
#pragma unroll
        for (int i = 0; i < LOADS; i++) {
            const int row = k_base + i * 32 + (tid >> 3);
            const int row_c = row < K ? row : K - 1;  // rows past K meet zero activations
            wld[i] = __builtin_nontemporal_load(
                reinterpret_cast<const u32x4*>(qweight + static_cast<size_t>(row_c) * nw + wcol_c));
        }
    }
    // scales and zero words of this wave's quantisation group: lanes 0..31 sixteen bytes of scales each,
    // lanes 32..39 sixteen bytes of zero words each (the other lanes repeat a valid address)
    u32x4 sld, zld;
    {
        const int krow = k_base + wave * WROWS;
        const int g = (krow < K ? krow : K - 1) >> group_shift;
        const int col = ct * kTileCols + (lane & 31) * 8;
        const int col_c = col < N ? col : N - 8;
        sld = *reinterpret_cast<const u32x4*>(scales + static_cast<size_t>(g) * N + col_c);
        const int zcol = ct * 32 + (lane & 7) * 4;
        const int zcol_c = zcol < nw ? zcol : nw - 4;
        zld = *reinterpret_cast<const u32x4*>(qzeros + static_cast<size_t>(g) * nw + zcol_c);
    }
    // activations: piece e = (row m, eight consecutive k); rows past M and k past K are zeros
    u32x4 xld[XPASSES];
    bool x_live[XPASSES];
#pragma unroll
    for (int ps = 0; ps < XPASSES; ps++) {
        const int e = tid + ps * kWideThreads;
        const int m = e / (KB / 8);
        const int k = k_base + (e % (KB / 8)) * 8;
        const int mc = m < M ? m : M - 1;
        const int kc = k < K ? k : K - 8;
        xld[ps] = *reinterpret_cast<const u32x4*>(x + static_cast<size_t>(mc) * K + kc);
        x_live[ps] = m < M && k < K;
    }

    // ---- into LDS ----
    {
        u32x4* tile = reinterpret_cast<u32x4*>(s_block);
#pragma unroll
        for (int i = 0; i < LOADS; i++) tile[i * kWideThreads + tid] = wld[i];  // row (32 i + t / 8), bytes 16 (t % 8)
    }
    if (lane < 32) *reinterpret_cast<u32x4*>(&s_sc[wave][lane * 8]) = sld;
    else if (lane < 40) *reinterpret_cast<u32x4*>(&s_zw[wave][(lane - 32) * 4]) = zld;
#pragma unroll
    for (int ps = 0; ps < XPASSES; ps++) {
        const int e = tid + ps * kWideThreads;
        if (e < XPIECES) {
            const u32x4 zero = {0u, 0u, 0u, 0u};
            *reinterpret_cast<u32x4*>(&s_x[e / (KB / 8)][(e % (KB / 8)) * 8]) = x_live[ps] ? xld[ps] : zero;
        }
    }
    __syncthreads();

    // ---- operands back out of LDS in the MFMA layout, then the matrix products ----
    uint32_t w[KS][8][2];
    u32x4 xa[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        const int row0 = (wave * KS + ks) * kStepRows + 8 * b;
#pragma unroll
        for (int r = 0; r < 8; r++) {
            const u32x2 v = *reinterpret_cast<const u32x2*>(s_block + (row0 + r) * 128 + 8 * c);
            w[ks][r][0] = v.x;
            w[ks][r][1] = v.y;
        }
        const u32x4 got = *reinterpret_cast<const u32x4*>(&s_x[c < ROWS ? c : 0][row0]);
        const bool live = c < ROWS;
        xa[ks] = u32x4{live ? got.x : 0u, live ? got.y : 0u, live ? got.z : 0u, live ? got.w : 0u};
    }

    const bf16x8 ones = as_bf16x8(0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u);
    const f32x4v zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    f32x4v xs;
    f32x4v acc[2][8];  // [word h][nibble p]
    const uint32_t magic = opaque_bf16_128_pair();
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        const bf16x8 a_op = as_bf16x8(xa[ks].x, xa[ks].y, xa[ks].z, xa[ks].w);
        xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_op, ones, ks == 0 ? zero4 : xs, 0, 0, 0);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint32_t bop[8][4];  // [nibble p][row pair]
#pragma unroll
            for (int rp = 0; rp < 4; rp++) {
                const uint32_t wa = w[ks][2 * rp][h];      // row 2rp   -> low half
                const uint32_t wb = w[ks][2 * rp + 1][h];  // row 2rp+1 -> high half
                const uint32_t lo = __builtin_amdgcn_perm(wb, wa, 0x05040100u);  // nibbles 0..3, both rows
                const uint32_t hi = __builtin_amdgcn_perm(wb, wa, 0x07060302u);  // nibbles 4..7
#pragma unroll
                for (int p = 0; p < 4; p++) {
                    bop[p][rp] = code_pair_to_bf16(p == 0 ? lo : lo >> (4 * p), magic);
                    bop[4 + p][rp] = code_pair_to_bf16(p == 0 ? hi : hi >> (4 * p), magic);
                }
            }
#pragma unroll
            for (int p = 0; p < 8; p++) {
                acc[h][p] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    a_op, as_bf16x8(bop[p][0], bop[p][1], bop[p][2], bop[p][3]), ks == 0 ? zero4 : acc[h][p], 0, 0, 0);
            }
        }
    }
    __syncthreads();  // every wave has read its part of the tile: the block now holds the waves' sums

    // ---- waves meet in LDS; thread t then owns tile column t ----
    float (*red)[MC][kTileCols] = reinterpret_cast<float (*)[MC][kTileCols]>(s_block);
    constexpr int VR = MC < 4 ? MC : 4;  // rows of the lane's four that exist at all
    float psum[ROWS];
#pragma unroll
    for (int rd = 0; rd < ROUNDS; rd++) {
        if (rd > 0) __syncthreads();  // the previous round has been read
        const int local0 = 4 * b - rd * MC;  // the lane's first row inside this round
        if (local0 >= 0 && local0 < MC) {
#pragma unroll
            for (int v = 0; v < VR; v++) {
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    f32x4* dst = reinterpret_cast<f32x4*>(&red[wave][local0 + v][16 * c + 8 * h]);
                    dst[0] = f32x4{acc[h][nibble_of(0)][v], acc[h][nibble_of(1)][v], acc[h][nibble_of(2)][v],
                                   acc[h][nibble_of(3)][v]};
                    dst[1] = f32x4{acc[h][nibble_of(4)][v], acc[h][nibble_of(5)][v], acc[h][nibble_of(6)][v],
                                   acc[h][nibble_of(7)][v]};
                }
                if (c == 0) xs_red[wave][local0 + v] = xs[v];
            }
        }
        __syncthreads();
        float sc[WAVES], zc[WAVES];
#pragma unroll
        for (int wv = 0; wv < WAVES; wv++) {
            sc[wv] = f16_bits_to_f32(s_sc[wv][tid]);
            zc[wv] = -(128.0f + static_cast<float>((s_zw[wv][tid >> 3] >> (4 * nibble_of(tid & 7))) & 0xFu));
        }
        float qv[MC][WAVES], xv[MC][WAVES];
#pragma unroll
        for (int v = 0; v < MC; v++) {
#pragma unroll
            for (int wv = 0; wv < WAVES; wv++) {
                qv[v][wv] = red[wv][v][tid];
                xv[v][wv] = xs_red[wv][v];
            }
        }
#pragma unroll
        for (int v = 0; v < MC; v++) {
            float total = 0.0f;
#pragma unroll
            for (int wv = 0; wv < WAVES; wv++) {
                total += sc[wv] * __builtin_fmaf(zc[wv], xv[v][wv], qv[v][wv]);
            }
            psum[rd * MC + v] = total;
        }
    }

    if constexpr (ROWS >= 4) {
        splitk_exchange_store_wide<ROWS>(psum, M, N, ct, kt, ktiles, partials, counters, y, &s_prev);
    } else {
        splitk_exchange_store<ROWS>(psum, 0, M, N, ct, kt, ktiles, ct, partials, counters, y, &s_prev);
    }
}

template <int KS, int MC, int ROUNDS>
inline void launch_awq_gemv_wide(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                                 const int32_t* qzeros, uint16_t* y, float* partials, uint32_t* counters,
                                 int M, int K, int N, int group_shift, int coltiles, int ktiles,
                                 hipStream_t stream) {
    dim3 grid(coltiles, ktiles, 1);
    dim3 block(kWideThreads, 1, 1);
    hipLaunchKernelGGL((awq_gemv_wide_kernel<KS, MC, ROUNDS>), grid, block, 0, stream, x,
                       reinterpret_cast<const uint32_t*>(qweight), scales,
                       reinterpret_cast<const uint32_t*>(qzeros), y, partials, counters, M, K, N,
                       group_shift, ktiles);
}

}  // namespace kx

#endif  // KX_AWQ_GEMV_WIDE_KERNEL_H
