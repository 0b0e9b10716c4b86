// Device side of the fused INT4 AWQ dequantise + GEMV (gfx950, wave64).
//
//   y[m,n] = sum_k x[m,k] * (q[k,n] - z[k/G,n]) * s[k/G,n]
//
// The packed stream is consumed as it lies in memory: qweight int32 [K, N/8], one word = eight
// columns of one row.  A lane owns one word column and RT consecutive rows (all inside one
// quantisation group), so that zero point and scale are applied once per lane and column:
//
//   y_part[n] = s[g,n] * ( sum_r q[k0+r,n] * x[k0+r]  -  z[g,n] * sum_r x[k0+r] )
//
// A wave covers 32 consecutive word columns (128 contiguous bytes of each row, 256 output
// columns) times two row slots; a workgroup stacks WAVES waves along K.  Row slots meet in LDS.
// Workgroups that share a column tile meet in a caller-provided workspace: each stores its 256
// partial sums, then bumps the tile's arrival counter; the workgroup that arrives last adds the
// partials in a fixed order (bitwise reproducible) and writes y.  Thread t of a workgroup owns
// tile column t in that exchange, so every store and load of partials is a contiguous 256 bytes
// per wave.
//
// The exchange itself is in kx_splitk_exchange.h.
#ifndef KX_AWQ_GEMV_KERNEL_H
#define KX_AWQ_GEMV_KERNEL_H

#include "kx_common.h"
#include "kx_splitk_exchange.h"

namespace kx {

constexpr int kWC = 32;                 // word columns per wave
static_assert(kWC * 8 == kTileCols, "a wave spans one column tile");
constexpr int kSlotsPerWave = kWave / kWC;


typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// The eight codes of a packed word as floats, indexed by column (0..7) inside the word.
// A byte 0x0q read as OCP fp8 (e4m3) is exactly q * 2^-9 for every q in 0..15 (subnormal below
// 8, normal from 8 on), so the packed fp8 -> fp32 conversion unpacks two codes per instruction.
// The factor 2^-9 is undone by kCodeScale when the group scale is applied.
constexpr float kCodeScale = 512.0f;

__device__ __forceinline__ void unpack_codes(uint32_t w, float (&q)[8]) {
    const uint32_t lo = w & 0x0F0F0F0Fu;         // nibbles 0, 2, 4, 6 in bytes 0..3
    const uint32_t hi = (w >> 4) & 0x0F0F0F0Fu;  // nibbles 1, 3, 5, 7
    const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8(lo, false);
    const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8(lo, true);
    const f32x2 c = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false);
    const f32x2 d = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
    q[order_of(0)] = a.x;
    q[order_of(2)] = a.y;
    q[order_of(4)] = b.x;
    q[order_of(6)] = b.y;
    q[order_of(1)] = c.x;
    q[order_of(3)] = c.y;
    q[order_of(5)] = d.x;
    q[order_of(7)] = d.y;
}

template <int WAVES, int RT, int MB>
__global__ __launch_bounds__(WAVES * kWave) void awq_gemv_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    uint16_t* __restrict__ y, float* __restrict__ partials, uint32_t* __restrict__ counters,
    int M, int K, int N, int group, int coltiles, int ktiles) {
    constexpr int SLOTS = WAVES * kSlotsPerWave;
    constexpr int KB = SLOTS * RT;
    static_assert(RT % 8 == 0, "a lane reads its activations in 16-byte pieces");

    __shared__ __attribute__((aligned(16))) float red[WAVES][kTileCols];

    const int tid = threadIdx.x;
    const int ct = blockIdx.x % coltiles;
    const int kt = blockIdx.x / coltiles;
    const int m0 = blockIdx.y * MB;
    const int nw = N >> 3;

    const int wc = tid % kWC;       // word column inside the tile
    const int slot = tid / kWC;     // row slot inside the workgroup
    const int wcg = ct * kWC + wc;  // word column in the matrix
    const int k0 = kt * KB + slot * RT;
    const bool active = (wcg < nw) && (k0 < K);

    float acc[MB][8];
#pragma unroll
    for (int m = 0; m < MB; m++) {
#pragma unroll
        for (int c = 0; c < 8; c++) acc[m][c] = 0.0f;
    }

    if (active) {
        // Small, cache-resident operands first, then every weight load of this lane, all of them
        // issued before anything is consumed: loads return in order, so the arithmetic on row r
        // can start while rows r+1.. are still in flight.
        const int g = k0 / group;
        const uint32_t zw = qzeros[static_cast<size_t>(g) * nw + wcg];
        const uint4 sraw = *reinterpret_cast<const uint4*>(scales + static_cast<size_t>(g) * N + 8 * wcg);
        uint4 xraw[MB][RT / 8];
#pragma unroll
        for (int m = 0; m < MB; m++) {
#pragma unroll
            for (int r8 = 0; r8 < RT / 8; r8++) {
                xraw[m][r8] = (m0 + m < M)
                    ? *reinterpret_cast<const uint4*>(x + static_cast<size_t>(m0 + m) * K + k0 + 8 * r8)
                    : make_uint4(0u, 0u, 0u, 0u);
            }
        }
        uint32_t w[RT];
        const uint32_t* wp = qweight + static_cast<size_t>(k0) * nw + wcg;
#pragma unroll
        for (int r = 0; r < RT; r++) {
            w[r] = __builtin_nontemporal_load(wp + static_cast<size_t>(r) * nw);
        }
        // keep the scheduler from sinking loads below the first use of an earlier one
        __builtin_amdgcn_sched_barrier(0);

        float xsum[MB];
#pragma unroll
        for (int m = 0; m < MB; m++) xsum[m] = 0.0f;

#pragma unroll
        for (int r8 = 0; r8 < RT; r8 += 8) {
            float xs[MB][8];
#pragma unroll
            for (int m = 0; m < MB; m++) {
                const uint4 xr = xraw[m][r8 / 8];
                const uint32_t xw[4] = {xr.x, xr.y, xr.z, xr.w};
#pragma unroll
                for (int r = 0; r < 8; r++) {
                    const uint32_t bits = (r & 1) ? (xw[r >> 1] & 0xffff0000u) : (xw[r >> 1] << 16);
                    xs[m][r] = __uint_as_float(bits);
                    xsum[m] += xs[m][r];
                }
            }
#pragma unroll
            for (int r = 0; r < 8; r++) {
                float q[8];
                unpack_codes(w[r8 + r], q);
#pragma unroll
                for (int m = 0; m < MB; m++) {
#pragma unroll
                    for (int c = 0; c < 8; c++) acc[m][c] = __builtin_fmaf(q[c], xs[m][r], acc[m][c]);
                }
            }
        }

        // zero point and scale, once per lane and column
        float z[8];
        unpack_codes(zw, z);
        const uint32_t sw[4] = {sraw.x, sraw.y, sraw.z, sraw.w};
        float s[8];
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const uint16_t bits = static_cast<uint16_t>((c & 1) ? (sw[c >> 1] >> 16) : (sw[c >> 1] & 0xffffu));
            s[c] = f16_bits_to_f32(bits) * kCodeScale;  // power of two: exact
        }
#pragma unroll
        for (int m = 0; m < MB; m++) {
#pragma unroll
            for (int c = 0; c < 8; c++) {
                acc[m][c] = s[c] * __builtin_fmaf(-z[c], xsum[m], acc[m][c]);
            }
        }
    }

    // The two row slots of a wave meet through a lane exchange, the waves of the workgroup in
    // LDS (one activation row at a time); afterwards thread t < 256 owns tile column t.
    static_assert(kSlotsPerWave == 2, "the lane exchange below pairs lane l with lane l + 32");
    static_assert(WAVES * kWave >= kTileCols, "one thread per tile column");
    const int wave = tid / kWave;
    const int lane = tid % kWave;
    float psum[MB];
#pragma unroll
    for (int m = 0; m < MB; m++) {
#pragma unroll
        for (int c = 0; c < 8; c++) acc[m][c] += __shfl_xor(acc[m][c], 32, kWave);
        if (m > 0) __syncthreads();  // the previous row has been read
        if (lane < kWC) {
            f32x4* dst = reinterpret_cast<f32x4*>(&red[wave][8 * lane]);
            dst[0] = f32x4{acc[m][0], acc[m][1], acc[m][2], acc[m][3]};
            dst[1] = f32x4{acc[m][4], acc[m][5], acc[m][6], acc[m][7]};
        }
        __syncthreads();
        psum[m] = 0.0f;
        if (tid < kTileCols) {
            float v[WAVES];
#pragma unroll
            for (int u = 0; u < WAVES; u++) v[u] = red[u][tid];
#pragma unroll
            for (int u = 0; u < WAVES; u++) psum[m] += v[u];
        }
    }

    __shared__ uint32_t s_prev;
    splitk_exchange_store<MB>(psum, m0, M, N, ct, kt, ktiles, blockIdx.y * coltiles + ct, partials, counters, y,
                              &s_prev);
}

template <int WAVES, int RT, int MB>
inline void launch_awq_gemv(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                            const int32_t* qzeros, uint16_t* y, float* partials, uint32_t* counters,
                            int M, int K, int N, int group, int coltiles, int ktiles, int mtiles,
                            hipStream_t stream) {
    dim3 grid(coltiles * ktiles, mtiles, 1);
    dim3 block(WAVES * kWave, 1, 1);
    hipLaunchKernelGGL((awq_gemv_kernel<WAVES, RT, MB>), grid, block, 0, stream, x,
                       reinterpret_cast<const uint32_t*>(qweight), scales,
                       reinterpret_cast<const uint32_t*>(qzeros), y, partials, counters, M, K, N,
                       group, coltiles, ktiles);
}

}  // namespace kx

#endif  // KX_AWQ_GEMV_KERNEL_H
