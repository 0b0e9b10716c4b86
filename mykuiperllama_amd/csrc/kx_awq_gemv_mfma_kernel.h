// Fused INT4 AWQ dequantise + GEMV on the matrix cores (gfx950, v_mfma_f32_16x16x32_bf16), M <= 16.
//
//   y[m,n] = sum_k x[m,k] * (q[k,n] - z[k/G,n]) * s[k/G,n]
//
// One MFMA multiplies A = activations (16 rows m x 32 k) by B = weights (32 k x 16 columns n) into a
// 16 x 16 fp32 tile.  Lane l of the wave supplies, for both operands, the eight k values
// 8*(l/16) .. 8*(l/16)+7 of row / column l%16, and receives D[4*(l/16)+v][l%16], v = 0..3.
//
// A lane (c = l%16, b = l/16) loads the two packed words (c-th pair of the tile's 32 word columns)
// of the eight rows 8b .. 8b+7 of a 32-row step: sixteen columns x eight rows of codes.  Nibble p of
// word h of those eight rows is exactly the B operand of column 8*(2c+h) + ORDER[p], so sixteen
// MFMAs per step - one per (h, p) - cover the lane's sixteen columns, all with the same A operand,
// which is a plain 16-byte load of x.  A code becomes a bf16 by OR-ing it into the mantissa of
// 128.0 (0x4300 | q = 128 + q, exact), two rows per register; the +128 joins the zero point:
//
//   sum_k x*(q - z) = sum_k x*(128 + q)  -  (128 + z) * sum_k x
//
// and sum_k x comes out of one more MFMA against a B operand of ones, in the same register layout.
// Raw sums of the waves of a workgroup meet in LDS; the thread that owns a column applies zero
// point and scale once per wave (a wave never straddles a quantisation group: groups are powers of
// two here and the host picks KS so that KS*32 divides the group) and takes part in the split-K exchange.
//
// Cost per weight: one VALU operation to build the operand (two byte permutes, three shifts and
// eight and/or pairs per sixteen weights) and 1/512 of an MFMA, whatever M is.
//
// The activations may be produced on the way in (PRO: SwiGLU of two tensors, or an RMSNorm whose sum of
// squares arrives per 256 columns) and the result may be added to a residual stream on the way out (EPI),
// with the arithmetic and rounding points of the stand-alone kernels.  A produced activation is staged
// in LDS as bf16, the workgroup's K range of every row, and the A operand is read from there.
#ifndef KX_AWQ_GEMV_MFMA_KERNEL_H
#define KX_AWQ_GEMV_MFMA_KERNEL_H

#include "kx_common.h"
#include "kx_gemv_fused.h"
#include "kx_rope.h"
#include "kx_splitk_exchange.h"

namespace kx {

constexpr int kStepRows = 32;  // rows of K per MFMA step

// Column (0..7) inside a word -> nibble that holds it (inverse of order_of).
__host__ __device__ constexpr int nibble_of(int col) {
    return (col & 1) ? 4 + (col >> 1) : (col >> 1);
}

// Two bf16 128.0 in a register whose value the compiler cannot see.  (v & 0x000F000F) | magic then
// selects as one v_and_or_b32 (a literal and a register); with two literals it would be split into
// v_and + v_or.  The conversion itself stays ordinary C so that the compiler keeps track of the
// registers the matrix instructions are still reading.
__device__ __forceinline__ uint32_t opaque_bf16_128_pair() {
    uint32_t out;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(out));
    return out;
}

__device__ __forceinline__ uint32_t code_pair_to_bf16(uint32_t v, uint32_t magic) {
    return (v & 0x000F000Fu) | magic;
}

// Eight consecutive bf16 of a 16-byte piece as floats, and back (round to nearest even).
__device__ __forceinline__ void bf16x8_to_f32(const uint4& v, float (&f)[8]) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] = __uint_as_float((i & 1) ? (w[i >> 1] & 0xffff0000u) : (w[i >> 1] << 16));
}
__device__ __forceinline__ uint4 f32_to_bf16x8(const float (&f)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        w[i] = static_cast<uint32_t>(f32_to_bf16(f[2 * i])) | (static_cast<uint32_t>(f32_to_bf16(f[2 * i + 1])) << 16);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// KS: consecutive 32-row steps per wave (they must share a quantisation group);
// MC: activation rows a workgroup reduces per LDS round (1, 2, 4 or 8); ROUNDS: 2 for M > 8, else 1.
// With a prologue, `x` is not read: fi.a / fi.b (/ fi.gain) are 16-byte aligned, fi.ld a multiple of eight.
template <int WAVES, int KS, int MC, int ROUNDS, int PRO = kProNone, int EPI = kEpiStore>
__global__ __launch_bounds__(WAVES * kWave, 2) void awq_gemv_mfma_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    uint16_t* __restrict__ y, float* __restrict__ partials, uint32_t* __restrict__ counters,
    int M, int K, int N, int group_shift, int ktiles, FusedInput fi, ResidualTarget res, RopeTarget rope,
    size_t cache_stride) {
    constexpr int WROWS = KS * kStepRows;  // rows of K per wave
    constexpr int KB = WAVES * WROWS;      // rows of K per workgroup
    constexpr int ROWS = MC * ROUNDS;      // activation rows this kernel carries (>= M)
    constexpr int THREADS = WAVES * kWave;
    static_assert(THREADS >= kTileCols, "one thread per tile column");
    static_assert(PRO == kProNone || PRO == kProSwiGLU || PRO == kProPreNorm, "prologues of the matrix-core kernel");
    static_assert(EPI == kEpiStore || EPI == kEpiResidual || EPI == kEpiQkRope, "epilogues of the matrix-core kernel");
    constexpr bool STAGED = PRO != kProNone;
    // A staged row is the workgroup's K range plus 16 bytes, so that the rows a wave reads together
    // start in different banks.
    constexpr int XPITCH = KB + 8;
    constexpr int KPIECES = KB / 8;             // 16-byte pieces per staged row
    constexpr int PIECES = ROWS * KPIECES;
    constexpr int PPT = (PIECES + THREADS - 1) / THREADS;  // pieces a thread produces

    __shared__ __attribute__((aligned(16))) float red[WAVES][MC][kTileCols];
    __shared__ float xs_red[WAVES][MC];
    __shared__ uint32_t s_prev;
    __shared__ __attribute__((aligned(16))) uint16_t s_x[STAGED ? ROWS : 1][STAGED ? XPITCH : 8];
    __shared__ float s_inv[PRO == kProPreNorm ? ROWS : 1];

    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int lane = tid % kWave;
    const int c = lane % 16;  // column slot: word pair c of the tile, MFMA column c
    const int b = lane / 16;  // k block inside the step, D row block
    const int ct = blockIdx.x;  // column tile; x runs fastest, so neighbours in time are neighbours in N
    const int kt = blockIdx.y;
    const int nw = N >> 3;

    const int kwave = kt * KB + wave * WROWS;  // first row of this wave

    // The rotary epilogue (row m of the result belongs to sequence m): the workgroup that finishes a column
    // tile holds two heads of every row; wave w will take the (row, head) items w, w + WAVES, ...  Its
    // positions and the heads' gains are requested now, long before the epilogue needs them.
    constexpr int ROPE_ITEMS = (2 * ROWS + WAVES - 1) / WAVES;  // items per wave
    int rope_pos[EPI == kEpiQkRope ? ROPE_ITEMS : 1];
    uint16_t rope_ga[2], rope_gb[2];
    if constexpr (EPI == kEpiQkRope) {
#pragma unroll
        for (int i = 0; i < ROPE_ITEMS; i++) {
            const int r = (wave + i * WAVES) / 2;
            rope_pos[i] = rope.pos[r < M ? r : M - 1];
        }
        // both gains, then a select of values (a select between pointers ends up as a table in private memory)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const bool q_head = ct * (kTileCols / kHeadDim) + h < rope.n_q;
            const uint16_t qa = rope.q_gain[lane], qb = rope.q_gain[lane + 64];
            const uint16_t ka = rope.k_gain[lane], kb = rope.k_gain[lane + 64];
            rope_ga[h] = q_head ? qa : ka;
            rope_gb[h] = q_head ? qb : kb;
        }
    }

    // ---- operands of the activation prologue go out first: they are small, mostly cached, and the prologue
    // should run while the weights are still on their way ----
    // Piece e = tid + i * THREADS of the workgroup is (row e / KPIECES, elements 8 (e % KPIECES) .. + 7 of
    // the K range); addresses are clamped, what a clamped load brings is replaced by zeros.
    uint4 pa[STAGED ? PPT : 1], pb[STAGED ? PPT : 1];
    float tile_ss[PRO == kProPreNorm ? (ROWS + WAVES - 1) / WAVES : 1];
    if constexpr (STAGED) {
#pragma unroll
        for (int i = 0; i < PPT; i++) {
            const int e = tid + i * THREADS;
            const int pm = e / KPIECES;
            const int k = kt * KB + 8 * (e % KPIECES);
            const int mc = pm < M ? pm : M - 1;
            const int kc = k < K ? k : K - 8;
            const size_t at = static_cast<size_t>(mc) * fi.ld + kc;
            pa[i] = *reinterpret_cast<const uint4*>(fi.a + at);
            if constexpr (PRO == kProSwiGLU) pb[i] = *reinterpret_cast<const uint4*>(fi.b + at);
            else pb[i] = *reinterpret_cast<const uint4*>(fi.gain + kc);
        }
        if constexpr (PRO == kProPreNorm) {
            // wave w adds the tiles of rows w, w + WAVES, ...: lane = tile
#pragma unroll
            for (int rr = 0; rr < (ROWS + WAVES - 1) / WAVES; rr++) {
                const int m = wave + rr * WAVES;
                const int mc = m < M ? m : M - 1;
                const f32x4 qs = reinterpret_cast<const f32x4*>(fi.sumsq)[static_cast<size_t>(mc) * fi.sumsq_parts +
                                                                          (lane < fi.sumsq_parts ? lane : fi.sumsq_parts - 1)];
                tile_ss[rr] = ((qs.x + qs.y) + qs.z) + qs.w;  // the order that defines a tile's sum
            }
        }
    }

    // ---- loads, all issued before anything is consumed ----
    // Every load is unconditional: an address that would fall outside is clamped to one inside, and
    // what it brings is either masked (activations) or lands in outputs that are never stored
    // (columns past N).  A load under a condition becomes a branch with a full wait behind it, and
    // a chain of those is a chain of memory round trips.
    //
    // Scale and zero point of the column this thread will own after the LDS round, one pair per
    // wave of the workgroup (a wave never straddles a quantisation group; waves that share a group
    // read the same address).
    const int own_col = ct * kTileCols + tid;
    const int own_ld = own_col < N ? own_col : N - 1;
    uint16_t s_bits[WAVES];
    uint32_t z_word[WAVES];
#pragma unroll
    for (int wv = 0; wv < WAVES; wv++) {
        const int krow = kt * KB + wv * WROWS;
        const int g = (krow < K ? krow : K - 1) >> group_shift;  // rows past K meet zero activations
        s_bits[wv] = scales[static_cast<size_t>(g) * N + own_ld];
        z_word[wv] = qzeros[static_cast<size_t>(g) * nw + (own_ld >> 3)];
    }
    // The A operand: row c of the activations, whether or not column slot c holds weights.  Rows
    // past M and steps past K (K is a multiple of 32: a step is all in or all out) are zeros.
    uint4 xa[KS];
    const int x_row = c < M ? c : M - 1;
    if constexpr (!STAGED) {
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int kstep = kwave + ks * kStepRows;
            const int kld = kstep < K ? kstep : K - kStepRows;
            const uint4 got = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(x_row) * K + kld + 8 * b);
            const bool live = c < M && kstep < K;
            xa[ks] = make_uint4(live ? got.x : 0u, live ? got.y : 0u, live ? got.z : 0u, live ? got.w : 0u);
        }
    }
    // The lane's two word columns, eight rows per step, both words in one load: the host sends only
    // N that are multiples of sixteen here, so word rows are 8-byte aligned.
    uint32_t w[KS][8][2];
    const int wc_first = ct * 32 + 2 * c;
    const int wc0 = wc_first < nw ? wc_first : nw - 2;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        const int kstep = kwave + ks * kStepRows;
        const int k0 = (kstep < K ? kstep : K - kStepRows) + 8 * b;  // first of the lane's eight rows
        const uint32_t* wp = qweight + static_cast<size_t>(k0) * nw + wc0;
#pragma unroll
        for (int r = 0; r < 8; r++) {
            const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(wp + static_cast<size_t>(r) * nw));
            w[ks][r][0] = v.x;
            w[ks][r][1] = v.y;
        }
    }
    __builtin_amdgcn_sched_barrier(0);
#if defined(KX_ABLATE) && KX_ABLATE == 2
    if (!STAGED && ktiles > 1) {  // profiling build: loads only - fold what arrived into one word and leave
        uint32_t f = 0;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            f ^= xa[ks].x ^ xa[ks].y ^ xa[ks].z ^ xa[ks].w;
#pragma unroll
            for (int r = 0; r < 8; r++) f ^= w[ks][r][0] ^ w[ks][r][1];
        }
#pragma unroll
        for (int wv = 0; wv < WAVES; wv++) f ^= s_bits[wv] ^ z_word[wv];
        if (f == 0x9E3779B9u) partials[tid] = 1.0f;
        return;
    }
#endif

    // ---- the activation prologue: produce the staged rows, then read the A operand back ----
    if constexpr (STAGED) {
        if constexpr (PRO == kProPreNorm) {
#pragma unroll
            for (int rr = 0; rr < (ROWS + WAVES - 1) / WAVES; rr++) {
                const int m = wave + rr * WAVES;
                const float total = wave_sum(lane < fi.sumsq_parts ? tile_ss[rr] : 0.0f);
                if (lane == 0 && m < ROWS) s_inv[m] = 1.0f / sqrtf(total / static_cast<float>(K) + fi.eps);
            }
            lds_barrier();
        }
#pragma unroll
        for (int i = 0; i < PPT; i++) {
            const int e = tid + i * THREADS;
            const int pm = e / KPIECES;
            const int kp = e % KPIECES;
            if (pm < ROWS) {
                float av[8], bv[8], out[8];
                bf16x8_to_f32(pa[i], av);
                bf16x8_to_f32(pb[i], bv);
                const bool live = pm < M && kt * KB + 8 * kp < K;  // K is a multiple of eight: a piece is all in or all out
                if constexpr (PRO == kProSwiGLU) {
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const float act = silu_rounded_to_bf16(av[j]);
                        out[j] = live ? act * bv[j] : 0.0f;
                    }
                } else {
                    const float inv = s_inv[pm];
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        out[j] = live ? bv[j] * bf16_to_f32(f32_to_bf16(av[j] * inv)) : 0.0f;
                    }
                }
                *reinterpret_cast<uint4*>(&s_x[pm][8 * kp]) = f32_to_bf16x8(out);
            }
        }
        lds_barrier();
        const int s_row = c < ROWS ? c : ROWS - 1;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const uint4 got = *reinterpret_cast<const uint4*>(&s_x[s_row][(wave * KS + ks) * kStepRows + 8 * b]);
            const bool live = c < M;  // rows M .. ROWS-1 and elements past K were staged as zeros
            xa[ks] = make_uint4(live ? got.x : 0u, live ? got.y : 0u, live ? got.z : 0u, live ? got.w : 0u);
        }
    }

    // ---- matrix products ----
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
        // a step is worked through while the loads of the later steps are still in flight
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- waves meet in LDS; thread t < 256 then owns tile column t ----
    // A round carries MC activation rows; a lane holds D rows 4b .. 4b+3 and joins the round they fall in.
    constexpr int VR = MC < 4 ? MC : 4;  // rows of the lane's four that exist at all
    float psum[ROWS];
#pragma unroll
    for (int rd = 0; rd < ROUNDS; rd++) {
        if (rd > 0) __syncthreads();  // the previous round has been read
        const int local0 = 4 * b - rd * MC;  // the lane's first row inside this round
        if (local0 >= 0 && local0 < MC) {
            // the lane's sixteen columns are 16c .. 16c+15
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
        if (tid < kTileCols) {
            float sc[WAVES], zc[WAVES];
#pragma unroll
            for (int wv = 0; wv < WAVES; wv++) {
                sc[wv] = f16_bits_to_f32(s_bits[wv]);
                zc[wv] = -(128.0f + static_cast<float>((z_word[wv] >> (4 * nibble_of(own_col & 7))) & 0xFu));
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
    }

#if defined(KX_ABLATE) && KX_ABLATE >= 1 && KX_ABLATE <= 3
    if (ktiles > 1) {  // profiling build: no exchange - every workgroup leaves its partial sums and is done
        if (tid < kTileCols && own_col < N) partials[static_cast<size_t>(kt) * M * N + own_col] = psum[0];
        return;
    }
#endif
    if constexpr (EPI == kEpiResidual || EPI == kEpiQkRope) {
        static_assert(THREADS == kTileCols, "these epilogues are laid out for 256 threads");
        // Thread t ends up with the finished sums of tile column t, every row; the residual rows are
        // requested as soon as the workgroup knows that it is the one to finish.
        float sum[ROWS];
        uint16_t rin[EPI == kEpiResidual ? ROWS : 1];
        auto load_residual = [&] {
            if constexpr (EPI == kEpiResidual) {
#pragma unroll
                for (int r = 0; r < ROWS; r++) rin[r] = res.in[static_cast<size_t>(r < M ? r : M - 1) * N + own_ld];
            }
        };
        if constexpr (ROWS >= 4) {
            // the wide read-back hands out two columns and half of the rows per thread: through LDS (the
            // reduction buffer, free again) to one column and every row per thread
            float* s_sum = &red[0][0][0];
            static_assert(WAVES * MC >= ROWS, "the reduction buffer holds a tile of finished sums");
            if (ktiles == 1) {
                load_residual();
#pragma unroll
                for (int r = 0; r < ROWS; r++) sum[r] = psum[r];
            } else {
                constexpr int HALF = ROWS / 2;
                float lo[HALF], hi[HALF];
                if (!splitk_exchange_sum_wide<ROWS>(psum, lo, hi, M, N, ct, kt, ktiles, partials, counters, &s_prev,
                                                    load_residual)) {
                    return;
                }
                const int row0 = (tid / (kTileCols / 2)) * HALF;
#pragma unroll
                for (int i = 0; i < HALF; i++) {
                    *reinterpret_cast<f32x2*>(&s_sum[(row0 + i) * kTileCols + 2 * (tid % (kTileCols / 2))]) = f32x2{lo[i], hi[i]};
                }
                __syncthreads();
#pragma unroll
                for (int r = 0; r < ROWS; r++) sum[r] = s_sum[r * kTileCols + tid];
            }
        } else if constexpr (EPI == kEpiResidual) {
            // every wave of 64 columns finishes for itself: the epilogue below needs nothing from the other waves
            load_residual();
            if (!splitk_exchange_sum_per_wave_rows<ROWS>(psum, sum, M, N, ct, kt, ktiles, partials, counters)) return;
        } else {
            if (!splitk_exchange_sum<ROWS>(psum, sum, 0, M, N, ct, kt, ktiles, ct, partials, counters, &s_prev)) return;
        }
        if constexpr (EPI == kEpiQkRope) {
            // The finished rows, rounded to bf16 as a separate GEMV would store them, go through LDS so that a
            // wave holds elements i and i + 64 of a head in lane i, the layout of the per-head routine.
            __shared__ uint16_t s_rows[ROWS][kTileCols];
#pragma unroll
            for (int r = 0; r < ROWS; r++) s_rows[r][tid] = f32_to_bf16(sum[r]);
            __syncthreads();
#pragma unroll
            for (int i = 0; i < ROPE_ITEMS; i++) {
                const int item = wave + i * WAVES;
                const int r = item / 2;
                const int h = item % 2;
                if (r < M) {  // the same in every lane of the wave
                    RopeTarget t = rope;
                    t.q_out += static_cast<size_t>(r) * rope.n_q * kHeadDim;
                    t.k_cache += static_cast<size_t>(r) * cache_stride;
                    t.v_cache += static_cast<size_t>(r) * cache_stride;
                    qk_norm_rope_head_with(s_rows[r][h * kHeadDim + lane], s_rows[r][h * kHeadDim + lane + 64],
                                           ct * (kTileCols / kHeadDim) + h, lane, t, rope_pos[i], rope_ga[h], rope_gb[h]);
                }
            }
        } else {
            // a wave is a quarter of the tile: its sum of squares of every row goes out as it is
            const bool col_ok = own_col < N;
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                float rv = 0.0f;
                if (col_ok && r < M) {
                    const float o = bf16_to_f32(f32_to_bf16(sum[r]));  // the projection's output is a bf16 tensor
                    const uint16_t rbits = f32_to_bf16(bf16_to_f32(rin[r]) + o);
                    res.out[static_cast<size_t>(r) * N + own_col] = rbits;
                    rv = bf16_to_f32(rbits);
                }
                const float q = wave_sum(rv * rv);
                if (lane == 0 && r < M) {
                    res.sumsq[(static_cast<size_t>(r) * gridDim.x + ct) * (kTileCols / kWave) + wave] = q;
                }
            }
        }
    } else if constexpr (ROWS >= 4) {
        static_assert(THREADS == kTileCols, "the wide exchange is laid out for 256 threads");
        splitk_exchange_store_wide<ROWS>(psum, M, N, ct, kt, ktiles, partials, counters, y, &s_prev);
    } else {
        // one or two activation rows: every wave of 64 columns is an exchange of its own
        float sum[ROWS];
        if (!splitk_exchange_sum_per_wave_rows<ROWS>(psum, sum, M, N, ct, kt, ktiles, partials, counters)) return;
        if (own_col < N) {
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                if (r < M) y[static_cast<size_t>(r) * N + own_col] = f32_to_bf16(sum[r]);
            }
        }
    }
}

template <int WAVES, int KS, int MC, int ROUNDS, int PRO = kProNone, int EPI = kEpiStore>
inline void launch_awq_gemv_mfma(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                                 const int32_t* qzeros, uint16_t* y, float* partials, uint32_t* counters,
                                 int M, int K, int N, int group_shift, int coltiles, int ktiles,
                                 hipStream_t stream, const FusedInput& fi = FusedInput{},
                                 const ResidualTarget& res = ResidualTarget{}, const RopeTarget& rope = RopeTarget{},
                                 size_t cache_stride = 0) {
    dim3 grid(coltiles, ktiles, 1);
    dim3 block(WAVES * kWave, 1, 1);
    hipLaunchKernelGGL((awq_gemv_mfma_kernel<WAVES, KS, MC, ROUNDS, PRO, EPI>), grid, block, 0, stream, x,
                       reinterpret_cast<const uint32_t*>(qweight), scales,
                       reinterpret_cast<const uint32_t*>(qzeros), y, partials, counters, M, K, N,
                       group_shift, ktiles, fi, res, rope, cache_stride);
}

}  // namespace kx

#endif  // KX_AWQ_GEMV_MFMA_KERNEL_H
