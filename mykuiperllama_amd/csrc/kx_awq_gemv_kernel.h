// Device side of the fused INT4 AWQ dequantise + GEMV (gfx950, wave64).
//
//   y[m,n] = sum_k x[m,k] * (q[k,n] - z[k/G,n]) * s[k/G,n]
//
// The packed stream is consumed as it lies in memory: qweight int32 [K, N/8], one word = eight
// columns of one row.  A lane owns one word column and RT consecutive rows (all inside one
// quantisation group), so that zero point and scale are applied once per lane and column.  Codes
// enter the arithmetic as bf16 numbers 16 + q, two rows per dot-product instruction:
//
//   y_part[n] = s[g,n] * ( sum_r (16 + q[k0+r,n]) * x[k0+r]  -  (16 + z[g,n]) * sum_r x[k0+r] )
//
// A wave covers 32 consecutive word columns (128 contiguous bytes of each row, 256 output
// columns) times two row slots; a workgroup stacks WAVES waves along K.  All row slots of a
// workgroup meet in LDS.
// Workgroups that share a column tile meet in a caller-provided workspace: each stores its 256
// partial sums, then bumps the tile's arrival counter; the workgroup that arrives last adds the
// partials in a fixed order (bitwise reproducible) and writes y.  Thread t of a workgroup owns
// tile column t in that exchange, so every store and load of partials is a contiguous 256 bytes
// per wave.
//
// The exchange itself is in kx_splitk_exchange.h.
#ifndef KX_AWQ_GEMV_KERNEL_H
#define KX_AWQ_GEMV_KERNEL_H

#include "kx_attn_merge.h"
#include "kx_common.h"
#include "kx_gemv_fused.h"
#include "kx_rope.h"
#include "kx_splitk_exchange.h"

namespace kx {

constexpr int kWC = 32;                 // word columns per wave
static_assert(kWC * 8 == kTileCols, "a wave spans one column tile");
constexpr int kSlotsPerWave = kWave / kWC;


typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// The eight codes of a packed word as floats times 2^-9, indexed by column (0..7) inside the word;
// used for the zero points, once per lane.  A byte 0x0q read as OCP fp8 (e4m3) is exactly q * 2^-9
// for every q in 0..15 (subnormal below 8, normal from 8 on), so the packed fp8 -> fp32 conversion
// unpacks two codes per instruction; kCodeScale undoes the factor.
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

constexpr float kCodeOffset = 16.0f;

// Two bf16 16.0 in a register whose value the compiler cannot see, so that (v & mask) | magic
// selects as one v_and_or_b32 (a literal and a register) instead of v_and + v_or.
__device__ __forceinline__ uint32_t opaque_bf16_pair_of_16() {
    uint32_t out;
    asm volatile("v_mov_b32 %0, 0x41804180" : "=v"(out));
    return out;
}

// codes at bits 3..6 of each half -> bf16 pair (16 + q_lo, 16 + q_hi)
__device__ __forceinline__ uint32_t code_pair_plus16(uint32_t v, uint32_t magic) {
    return (v & 0x00780078u) | magic;
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

// a.x * b.x + a.y * b.y + c in fp32, operands as packed bf16 pairs
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
    bf16x2_t va, vb;
    __builtin_memcpy(&va, &a, 4);
    __builtin_memcpy(&vb, &b, 4);
    return __builtin_amdgcn_fdot2_f32_bf16(va, vb, c, false);
}

template <int WAVES, int RT, int MB, int PRO, int EPI>
__global__ __launch_bounds__(WAVES * kWave) void awq_gemv_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    uint16_t* __restrict__ y, float* __restrict__ partials, uint32_t* __restrict__ counters,
    int M, int K, int N, int group, int group_shift, int coltiles, int ktiles, FusedInput fi, RopeTarget rope,
    ResidualTarget res) {
    constexpr int SLOTS = WAVES * kSlotsPerWave;
    constexpr int KB = SLOTS * RT;
    constexpr int THREADS = WAVES * kWave;
    constexpr bool STAGED = PRO != kProNone;
    constexpr bool NORM = PRO == kProAddNorm || PRO == kProAddNormLong;
    constexpr int NCH = PRO == kProAddNormLong ? kNormChunks : 1;
    constexpr bool MERGE = PRO == kProAttnMerge;
    constexpr bool PRENORM = PRO == kProPreNorm;
    static_assert(!PRENORM || MB == 1, "the pre-reduced norm serves one activation row");
    constexpr int HB = KB / kHeadDim > 0 ? KB / kHeadDim : 1;     // heads in the workgroup's K range
    constexpr int EPT = kMergeParts * KB / THREADS;               // (part, row) elements a thread merges
    static_assert(!MERGE || (MB == 1 && KB % kHeadDim == 0 && EPT * THREADS == kMergeParts * KB && HB <= WAVES),
                  "the attention merge serves one activation row and whole heads");
    static_assert(RT % 8 == 0, "a lane reads its activations in 16-byte pieces");
    static_assert(KB <= THREADS, "one staging thread per row of the workgroup's K range");

    __shared__ __attribute__((aligned(16))) float red[WAVES * kSlotsPerWave][kTileCols];
    __shared__ __attribute__((aligned(16))) uint16_t s_x[STAGED ? MB : 1][STAGED ? KB : 8];  // staged activations, bf16
    __shared__ float s_ss[NORM ? MB : 1][WAVES];
    __shared__ __attribute__((aligned(16))) float s_factor[MERGE ? HB : 1][MERGE ? kMergeParts * kMergeHold : 4];
    __shared__ float s_norm[MERGE ? HB : 1];
    __shared__ float s_mpart[MERGE ? kMergeParts : 1][MERGE ? KB : 1];

    // The pointers of the epilogue are fetched with the other kernel arguments: left to itself the compiler loads
    // them where they are first used, a scalar-memory round trip behind the reduction.
    asm volatile("" ::"s"(y), "s"(partials), "s"(counters));
    const int tid = threadIdx.x;
    // grid = (column tiles, K tiles, activation-row tiles): x runs fastest, so workgroups that start together read
    // neighbouring 128-byte pieces of the same rows, and no division stands in front of the first load
    const int ct = blockIdx.x;
    const int kt = blockIdx.y;
    const int m0 = blockIdx.z * MB;
    const int nw = N >> 3;

    const int wc = tid % kWC;       // word column inside the tile
    const int slot = tid / kWC;     // row slot inside the workgroup
    const int wcg = ct * kWC + wc;  // word column in the matrix
    const int k0 = kt * KB + slot * RT;
    const bool active = (wcg < nw) && (k0 < K);

    // Small operands of the epilogue and of the pre-reduced norm are requested first of all, so
    // that they have long arrived when they are needed (clamped addresses, masked use).
    uint16_t resid_pre = 0;
    if constexpr (EPI == kEpiResidual) {
        const int col = ct * kTileCols + tid % kTileCols;
        resid_pre = res.in[col < N ? col : N - 1];
    }
    int rope_pos = 0;
    uint16_t rope_gain_a = 0, rope_gain_b = 0;
    if constexpr (EPI == kEpiQkRope) {
        // what the wave that finishes head 2 ct + (tid / 128) will need, see the epilogue below
        const int head = ct * (kTileCols / kHeadDim) + ((tid % kTileCols) >> 7);
        // both gains, then a select of values: a select between pointers ends up as a table in private memory
        const bool q_head = head < rope.n_q;
        const uint16_t qa = rope.q_gain[tid % kWave], qb = rope.q_gain[tid % kWave + 64];
        const uint16_t ka = rope.k_gain[tid % kWave], kb = rope.k_gain[tid % kWave + 64];
        rope_gain_a = q_head ? qa : ka;
        rope_gain_b = q_head ? qb : kb;
        rope_pos = rope.pos[0];
    }
    float tile_ss = 0.0f;
    if constexpr (PRO == kProPreNorm) {
        const int part = tid % kWave;
        // four quarter sums per tile, added in the order that defines the tile's sum
        const f32x4 qs = reinterpret_cast<const f32x4*>(fi.sumsq)[part < fi.sumsq_parts ? part : fi.sumsq_parts - 1];
        tile_ss = ((qs.x + qs.y) + qs.z) + qs.w;
    }

    float acc[MB][8];
#pragma unroll
    for (int m = 0; m < MB; m++) {
#pragma unroll
        for (int c = 0; c < 8; c++) acc[m][c] = 0.0f;
    }

    // Operands of the activation prologue go out first: loads return in order, and the prologue
    // should run while the weights are still on their way.  Thread t produces row kt*KB + t.
    // Addresses are clamped instead of guarded so that the loads are straight-line code and all in
    // flight together; what a clamped load returns is masked where it is used.
    const int krow = kt * KB + tid;
    const bool stager = STAGED && tid < KB && krow < K;
    const bool has_b = PRO == kProSwiGLU || fi.b != nullptr;
    const uint16_t* b_src = has_b ? fi.b : fi.a;  // without a delta the second operand is read and ignored
    uint16_t own_a[MB], own_b[MB], own_gain = 0;
    uint4 row_a[NORM ? MB : 1][NCH], row_b[NORM ? MB : 1][NCH];
    float held[MERGE ? EPT : 1][MERGE ? kMergeHold : 1];
    MergeStats<kMergeStatsPerLane> stats;
    if constexpr (MERGE) {
        // element e of the workgroup = (part, row): row of the K range, chunks part, part + 4, ...
        const int G = fi.heads_per_kv;
        const size_t cstride = static_cast<size_t>(G) * kHeadDim;
#pragma unroll
        for (int i = 0; i < EPT; i++) {
            const int e = tid + i * THREADS;
            const int part = e / KB;
            const int rrow = kt * KB + e % KB;
            const int row_c = rrow < K ? rrow : K - 1;
            const int hq = row_c / kHeadDim;
            const float* po = fi.part_out + (static_cast<size_t>(hq / G) * fi.nchunks * G + hq % G) * kHeadDim +
                              row_c % kHeadDim;
#pragma unroll
            for (int j = 0; j < kMergeHold; j++) {
                const int c = part + j * kMergeParts;
                held[i][j] = po[(c < fi.nchunks ? c : fi.nchunks - 1) * cstride];
            }
        }
        // wave w prepares the factors of head w of the K range
        const int wave_id = tid / kWave;
        if (wave_id < HB) {
            const int hq0 = kt * HB + wave_id;
            const int hq = hq0 * kHeadDim < K ? hq0 : K / kHeadDim - 1;
            stats = attn_merge_load<kMergeStatsPerLane>(fi.part_ml + static_cast<size_t>(hq / G) * fi.nchunks * G * 2,
                                                        hq % G, G, fi.nchunks, tid % kWave);
        }
    }
    if constexpr (STAGED && !MERGE) {
        const int krow_c = krow < K ? krow : K - 1;
#pragma unroll
        for (int m = 0; m < MB; m++) {
            const int mrow = m0 + m < M ? m0 + m : M - 1;
            const size_t at = static_cast<size_t>(mrow) * fi.ld + krow_c;
            own_a[m] = fi.a[at];
            own_b[m] = b_src[at];
        }
        if constexpr (NORM || PRENORM) own_gain = fi.gain[krow_c];
    }
    if constexpr (NORM) {
        const int last_chunk = (K >> 3) - 1;
#pragma unroll
        for (int m = 0; m < MB; m++) {
            const int mrow = m0 + m < M ? m0 + m : M - 1;
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                const int c = tid + j * THREADS;
                const size_t at = static_cast<size_t>(mrow) * fi.ld + 8 * (c < last_chunk ? c : last_chunk);
                row_a[m][j] = *reinterpret_cast<const uint4*>(fi.a + at);
                row_b[m][j] = *reinterpret_cast<const uint4*>(b_src + at);
            }
        }
    }

    // Fixed-point exchange: what the unit of a column is made of (kx_splitk_exchange.h) is requested ahead of the
    // weights and summed while they are on their way.  Every wave that will own columns (threads 0..255) reads the
    // same sample of the activation row - eight spread-out runs of 128 bytes, 512 elements - and the scale of its
    // column in group 0; the wave sum needs no LDS and is the same bits in every workgroup of the launch.
    constexpr bool FIXED = EPI == kEpiStoreFixed;
    static_assert(!FIXED || (MB == 1 && PRO == kProNone), "the fixed-point exchange serves the plain one-row launch");
    FixedUnit fixed_unit{1.0f, 1.0f};
    u32x4 fixed_xs = {0u, 0u, 0u, 0u};
    uint16_t fixed_sref = 0;
    if constexpr (FIXED) {
        // every wave loads, also those that will own no column: a branch here would make every later wait a wait
        // for all loads
        const int pieces = K >> 3;                         // 16-byte pieces of the row, at least four (K >= 32)
        const int run = (tid % kWave) >> 3;                // eight runs of eight pieces
        const int pc = static_cast<int>((static_cast<long>(run) * pieces) >> 3) + (tid & 7);
        fixed_xs = *reinterpret_cast<const u32x4*>(x + 8 * (pc < pieces ? pc : pieces - 1));
        const int col = ct * kTileCols + tid % kTileCols;
        fixed_sref = scales[col < N ? col : N - 1];
    }
    // Small, cache-resident operands first, then every weight load of this lane, all of them
    // issued before anything is consumed: loads return in order, so the arithmetic on row r
    // can start while rows r+1.. are still in flight.
    // With a prologue the loads are not guarded either: a branch around them would make the wait
    // for the prologue's operands a wait for the weights as well.  Lanes outside the matrix read a
    // clamped address and take no part in the arithmetic.
    uint32_t zw = 0;
    uint4 sraw = make_uint4(0u, 0u, 0u, 0u);
    uint4 xraw[MB][RT / 8];
    uint32_t w[RT];
    constexpr bool CLAMPED = STAGED || FIXED;  // loads at clamped addresses instead of a branch around them
    if (CLAMPED || active) {
        const int ld_wcg = CLAMPED ? (wcg < nw ? wcg : nw - 1) : wcg;
        const int ld_k0 = CLAMPED ? (k0 < K ? k0 : K - RT) : k0;
        // power-of-two groups (the usual case) by a shift: a division is some forty instructions ahead of the loads
        const int g = group_shift >= 0 ? ld_k0 >> group_shift : ld_k0 / group;
        // On the plain launch scales and zero points carry the weights' streaming hint: measured + 1 % on the
        // seven-projection step; on the launches of the decode step the same hint cost 0.4 %.
        if constexpr (PRO == kProNone) {
            zw = __builtin_nontemporal_load(qzeros + static_cast<size_t>(g) * nw + ld_wcg);
            const u32x4 sv = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(scales + static_cast<size_t>(g) * N + 8 * ld_wcg));
            sraw = make_uint4(sv.x, sv.y, sv.z, sv.w);
        } else {
            zw = qzeros[static_cast<size_t>(g) * nw + ld_wcg];
            sraw = *reinterpret_cast<const uint4*>(scales + static_cast<size_t>(g) * N + 8 * ld_wcg);
        }
        if constexpr (!STAGED) {
#pragma unroll
            for (int m = 0; m < MB; m++) {
#pragma unroll
                for (int r8 = 0; r8 < RT / 8; r8++) {
                    // rows past M read row M - 1 and are zeroed: no branch between the loads
                    const int mrow = m0 + m < M ? m0 + m : M - 1;
                    const uint4 got = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(mrow) * K + ld_k0 + 8 * r8);
                    xraw[m][r8] = (m == 0 || m0 + m < M) ? got : make_uint4(0u, 0u, 0u, 0u);
                }
            }
        }
        if constexpr (STAGED) {
            // Buffer loads: the lane's offset is one register for all RT loads and the row's offset a scalar, so
            // the loads cost no vector ALU work (global loads take a 64-bit address each: two vector additions
            // per load in front of the prologue's arithmetic).  Measured on the decode step: 0.3 us per layer at
            // the 8B shape, 0.8 us at the 32B shape; the plain launch, which has nothing else to do while it
            // issues its loads, is 0.3 % slower with them and keeps global loads.  Rows past K read zeros.
            // The host keeps the packed weights of these launches below 2 GiB (32-bit offsets).
            const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<uint32_t*>(qweight), 0, static_cast<int>(static_cast<uint32_t>(static_cast<size_t>(K) * nw * 4)),
                0x00020000);
            const int voff = static_cast<int>((static_cast<size_t>(slot) * RT * nw + ld_wcg) * 4);
            const int sbase = __builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<size_t>(kt) * KB * nw * 4));
            constexpr int kStreaming = 2;  // the nt bit, as on the global loads
#pragma unroll
            for (int r = 0; r < RT; r++) {
                w[r] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, voff, sbase + r * nw * 4, kStreaming);
            }
        } else {
            const uint32_t* wp = qweight + static_cast<size_t>(ld_k0) * nw + ld_wcg;
#pragma unroll
            for (int r = 0; r < RT; r++) {
                w[r] = __builtin_nontemporal_load(wp + static_cast<size_t>(r) * nw);
            }
        }
        // keep the scheduler from sinking loads below the first use of an earlier one
        __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (FIXED) {
        const uint32_t pw[4] = {fixed_xs.x, fixed_xs.y, fixed_xs.z, fixed_xs.w};
        float xa = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; i++) xa = dot2_bf16(pw[i] & 0x7fff7fffu, 0x3F803F80u, xa);
        // the sample stands for the whole row: K / 512 elements per element read
        fixed_unit = fixed_unit_of(wave_sum(xa) * (static_cast<float>(K) * (1.0f / 512.0f)) *
                                   __builtin_fabsf(f16_bits_to_f32(fixed_sref)));
        // pinned here: left to itself the compiler sinks this arithmetic to its one use, behind the reduction
        asm volatile("" : "+v"(fixed_unit.unit), "+v"(fixed_unit.inv_unit));
        __builtin_amdgcn_sched_barrier(0);
    }
    // The rotation's sine and cosine while the weights are on their way: the vector unit has nothing to do yet,
    // and the wave that finishes a head finds them ready instead of working them out behind the exchange.
    float rope_sin = 0.0f, rope_cos = 1.0f;
    if constexpr (EPI == kEpiQkRope) {
        rope_angle(rope, rope_pos, tid % kWave, &rope_sin, &rope_cos);
        __builtin_amdgcn_sched_barrier(0);
    }
#if defined(KX_ABLATE) && KX_ABLATE == 2
    if constexpr (!STAGED) {
        if (ktiles > 1) {  // profiling build: loads only - fold what arrived into one word and leave
            uint32_t f = zw ^ sraw.x ^ sraw.y ^ sraw.z ^ sraw.w;
#pragma unroll
            for (int r = 0; r < RT; r++) f ^= w[r];
#pragma unroll
            for (int m = 0; m < MB; m++) {
#pragma unroll
                for (int r8 = 0; r8 < RT / 8; r8++) f ^= xraw[m][r8].x ^ xraw[m][r8].y ^ xraw[m][r8].z ^ xraw[m][r8].w;
            }
            if (f == 0x9E3779B9u) partials[tid] = 1.0f;
            return;
        }
    }
#endif

    if constexpr (MERGE) {
        const int wave_id = tid / kWave;
        if (wave_id < HB) {
            const float l = attn_merge_finish<kMergeStatsPerLane>(stats, s_factor[wave_id], kMergeHold, tid % kWave);
            if (tid % kWave == 0) s_norm[wave_id] = l;
        }
        lds_barrier();
#pragma unroll
        for (int i = 0; i < EPT; i++) {
            const int e = tid + i * THREADS;
            const int part = e / KB;
            const int row = e % KB;
            // The thread's kMergeHold factors lie side by side and chunks that do not exist carry factor 0, so
            // the sum is straight-line code: a test on the chunk count per step had been compiled to a branch
            // and an LDS read with a full wait per chunk, forty dependent LDS round trips per thread.
            static_assert(kMergeHold % 4 == 0, "the factors are read four at a time");
            const f32x4* f4 = reinterpret_cast<const f32x4*>(&s_factor[row / kHeadDim][part * kMergeHold]);
            float f[kMergeHold];
#pragma unroll
            for (int j4 = 0; j4 < kMergeHold / 4; j4++) {
                const f32x4 v = f4[j4];
                f[4 * j4] = v.x;
                f[4 * j4 + 1] = v.y;
                f[4 * j4 + 2] = v.z;
                f[4 * j4 + 3] = v.w;
            }
            float acc_m = 0.0f;
#pragma unroll
            for (int j = 0; j < kMergeHold; j++) acc_m = attn_merge_step(acc_m, held[i][j], f[j]);
            s_mpart[part][row] = acc_m;
        }
        lds_barrier();
        if (tid < KB) {
            const float total = (s_mpart[0][tid] + s_mpart[1][tid]) + (s_mpart[2][tid] + s_mpart[3][tid]);
            const float l = s_norm[tid / kHeadDim];
            const uint16_t xv = f32_to_bf16(l > 0.0f ? total / l : 0.0f);  // no position to attend to: zeros
            s_x[0][tid] = stager ? xv : static_cast<uint16_t>(0);
        }
        lds_barrier();
    }
    if constexpr (PRO == kProSwiGLU) {
        if (tid < KB) {
#pragma unroll
            for (int m = 0; m < MB; m++) {
                const float gt = bf16_to_f32(own_a[m]);
                const float act = silu_rounded_to_bf16(gt);
                const uint16_t xv = f32_to_bf16(act * bf16_to_f32(own_b[m]));
                s_x[m][tid] = (stager && m0 + m < M) ? xv : static_cast<uint16_t>(0);
            }
        }
        lds_barrier();
    }
    if constexpr (PRENORM) {
        if (tid < kWave) {
            const float total = wave_sum(tid < fi.sumsq_parts ? tile_ss : 0.0f);
            if (tid == 0) s_ss[0][0] = 1.0f / sqrtf(total / static_cast<float>(K) + fi.eps);
        }
        lds_barrier();
        if (tid < KB) {
            const float inv = s_ss[0][0];
            const float h = bf16_to_f32(own_gain) * bf16_to_f32(f32_to_bf16(bf16_to_f32(own_a[0]) * inv));
            s_x[0][tid] = stager ? f32_to_bf16(h) : static_cast<uint16_t>(0);
        }
        lds_barrier();
    }
    if constexpr (NORM) {
        // sum of squares of the whole updated row, in the order of the stand-alone norm kernel
#pragma unroll
        for (int m = 0; m < MB; m++) {
            float ss = 0.0f;
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                const uint32_t aw[4] = {row_a[m][j].x, row_a[m][j].y, row_a[m][j].z, row_a[m][j].w};
                const uint32_t bw[4] = {row_b[m][j].x, row_b[m][j].y, row_b[m][j].z, row_b[m][j].w};
                const bool valid = tid + j * THREADS < (K >> 3);
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float av = __uint_as_float((i & 1) ? (aw[i >> 1] & 0xffff0000u) : (aw[i >> 1] << 16));
                    const float bv = __uint_as_float((i & 1) ? (bw[i >> 1] & 0xffff0000u) : (bw[i >> 1] << 16));
                    // r = bf16(a + b); without a delta r = a, whose square a + 0 leaves unchanged
                    const float r = bf16_to_f32(f32_to_bf16(av + (has_b ? bv : 0.0f)));
                    ss += valid ? r * r : 0.0f;
                }
            }
            ss = wave_sum(ss);
            if (tid % kWave == 0) s_ss[m][tid / kWave] = ss;
        }
        lds_barrier();
        if (tid < KB) {
#pragma unroll
            for (int m = 0; m < MB; m++) {
                float total = 0.0f;
#pragma unroll
                for (int u = 0; u < WAVES; u++) total += s_ss[m][u];
                const float inv = 1.0f / sqrtf(total / static_cast<float>(K) + fi.eps);
                const uint16_t sum_bits = f32_to_bf16(bf16_to_f32(own_a[m]) + bf16_to_f32(own_b[m]));
                const uint16_t rbits = has_b ? sum_bits : own_a[m];
                const float r = bf16_to_f32(rbits);
                const float h = bf16_to_f32(own_gain) * bf16_to_f32(f32_to_bf16(r * inv));
                const bool live = stager && m0 + m < M;
                s_x[m][tid] = live ? f32_to_bf16(h) : static_cast<uint16_t>(0);
                if (ct == 0 && live && fi.r_out) {
                    fi.r_out[static_cast<size_t>(m0 + m) * K + krow] = rbits;
                }
            }
        }
        lds_barrier();
    }

    if (FIXED || active) {
        // Two rows at a time: the codes of rows k and k+1 of one column become a pair of bf16 numbers
        // 16 + q (exponent of 16.0, the code in the top four mantissa bits), the activations of the two
        // rows already lie in memory as such a pair, and one dot-product instruction does both
        // multiply-adds in fp32.  The offset is taken out again with the zero point:
        //   sum_k x (q - z) = sum_k x (16 + q)  -  (16 + z) sum_k x
        const uint32_t magic = opaque_bf16_pair_of_16();
        const uint32_t ones = 0x3F803F80u;  // bf16 (1, 1)
        float xsum[MB];
#pragma unroll
        for (int m = 0; m < MB; m++) xsum[m] = 0.0f;
        // Scale and 16 + zero point of the lane's eight columns: they arrived ahead of the weights, and what is
        // converted here does not stand between the last weight row and the reduction.  With 32 rows per lane the
        // sixteen registers this keeps across the loop cost more than the shorter tail gains (measured), and
        // the conversion stays behind the loop.
        // The fixed-point launch has no branch around its loads or its arithmetic: lanes outside the matrix work on
        // what their clamped addresses hold and contribute through a scale of zero.
        auto lane_scale = [&](float sc) { return (FIXED && !active) ? 0.0f : sc; };
        constexpr bool kConvertEarly = RT <= 16;
        float col_scale[8], col_zoff[8];
        if constexpr (kConvertEarly) {
            float z[8];
            unpack_codes(zw, z);
            const uint32_t sw[4] = {sraw.x, sraw.y, sraw.z, sraw.w};
#pragma unroll
            for (int c = 0; c < 8; c++) {
                const uint16_t bits = static_cast<uint16_t>((c & 1) ? (sw[c >> 1] >> 16) : (sw[c >> 1] & 0xffffu));
                col_scale[c] = lane_scale(f16_bits_to_f32(bits));
                col_zoff[c] = __builtin_fmaf(z[c], kCodeScale, kCodeOffset);  // 16 + z, exact
            }
            __builtin_amdgcn_sched_barrier(0);
        }

#pragma unroll
        for (int rp = 0; rp < RT / 2; rp++) {
            uint32_t xp[MB];
#pragma unroll
            for (int m = 0; m < MB; m++) {
                if constexpr (STAGED) {
                    xp[m] = *reinterpret_cast<const uint32_t*>(&s_x[m][slot * RT + 2 * rp]);
                } else {
                    const uint4 xr = xraw[m][rp / 4];
                    const uint32_t xw[4] = {xr.x, xr.y, xr.z, xr.w};
                    xp[m] = xw[rp % 4];
                }
                xsum[m] = dot2_bf16(xp[m], ones, xsum[m]);
            }
            const uint32_t wa = w[2 * rp], wb = w[2 * rp + 1];
            const uint32_t lo = __builtin_amdgcn_perm(wb, wa, 0x05040100u);  // nibbles 0..3 of both rows
            const uint32_t hi = __builtin_amdgcn_perm(wb, wa, 0x07060302u);  // nibbles 4..7
#pragma unroll
            for (int i = 0; i < 4; i++) {
                // nibble i sits at bits 4i of each half and goes to bits 3..6
                const uint32_t plo = code_pair_plus16(i == 0 ? lo << 3 : lo >> (4 * i - 3), magic);
                const uint32_t phi = code_pair_plus16(i == 0 ? hi << 3 : hi >> (4 * i - 3), magic);
#pragma unroll
                for (int m = 0; m < MB; m++) {
                    acc[m][order_of(i)] = dot2_bf16(plo, xp[m], acc[m][order_of(i)]);
                    acc[m][order_of(4 + i)] = dot2_bf16(phi, xp[m], acc[m][order_of(4 + i)]);
                }
            }
        }

        // zero point and scale, once per lane and column
        if constexpr (!kConvertEarly) {
            float z[8];
            unpack_codes(zw, z);
            const uint32_t sw[4] = {sraw.x, sraw.y, sraw.z, sraw.w};
#pragma unroll
            for (int c = 0; c < 8; c++) {
                const uint16_t bits = static_cast<uint16_t>((c & 1) ? (sw[c >> 1] >> 16) : (sw[c >> 1] & 0xffffu));
                col_scale[c] = lane_scale(f16_bits_to_f32(bits));
                col_zoff[c] = __builtin_fmaf(z[c], kCodeScale, kCodeOffset);  // 16 + z, exact
            }
        }
#pragma unroll
        for (int c = 0; c < 8; c++) {
#pragma unroll
            for (int m = 0; m < MB; m++) {
                acc[m][c] = col_scale[c] * __builtin_fmaf(-col_zoff[c], xsum[m], acc[m][c]);
            }
        }
    }

#if defined(KX_ABLATE) && KX_ABLATE == 3
    if constexpr (!STAGED) {
        if (ktiles > 1) {  // profiling build: loads and arithmetic - no reduction across lanes and waves, no exchange
            float f = 0.0f;
#pragma unroll
            for (int m = 0; m < MB; m++) {
#pragma unroll
                for (int c = 0; c < 8; c++) f += acc[m][c];
            }
            if (f == 12345.678f) partials[tid] = 1.0f;
            return;
        }
    }
#endif
    // The row slots of the workgroup meet in LDS (one activation row at a time); afterwards thread t < 256 owns
    // tile column t.  (A lane exchange between the two slots of a wave in front of the LDS round — a shuffle by
    // 32 lanes, itself an LDS round trip — halved the LDS traffic and cost 0.1 us per launch.)
    static_assert(kSlotsPerWave == 2, "the sum below pairs the two row slots of a wave");
    static_assert(WAVES * kWave >= kTileCols, "one thread per tile column");
    const int wave = tid / kWave;
    const int lane = tid % kWave;
    float psum[MB];
#pragma unroll
    for (int m = 0; m < MB; m++) {
        // every row slot leaves its eight sums in LDS; the two slots of a wave are added first, then the waves in
        // order (the grouping a lane exchange inside the wave followed by a sum over the waves would give)
        if (m > 0) __syncthreads();  // the previous row has been read
        {
            f32x4* dst = reinterpret_cast<f32x4*>(&red[slot][8 * wc]);
            dst[0] = f32x4{acc[m][0], acc[m][1], acc[m][2], acc[m][3]};
            dst[1] = f32x4{acc[m][4], acc[m][5], acc[m][6], acc[m][7]};
        }
        __syncthreads();
        psum[m] = 0.0f;
        if (tid < kTileCols) {
            float v[SLOTS];
#pragma unroll
            for (int u = 0; u < SLOTS; u++) v[u] = red[u][tid];
#pragma unroll
            for (int u = 0; u < WAVES; u++) psum[m] += v[2 * u] + v[2 * u + 1];
        }
    }

    __shared__ uint32_t s_prev;
#if defined(KX_ABLATE) && KX_ABLATE >= 1 && KX_ABLATE <= 3
    if (ktiles > 1) {  // profiling build: no exchange - every workgroup leaves its partial sums and is done
        const int col = ct * kTileCols + tid;
        if (tid < kTileCols && col < N) partials[static_cast<size_t>(kt) * M * N + col] = psum[0];
        return;
    }
#endif
    if constexpr (EPI == kEpiStoreFixed) {
        if (tid >= kTileCols) return;
        if (ktiles == 1) {
            const int col = ct * kTileCols + tid;
            if (col < N) store_result(y + col, f32_to_bf16(psum[0]));
            return;
        }
        splitk_exchange_store_fixed(psum[0], fixed_unit, N, ct, kt, ktiles,
                                    reinterpret_cast<unsigned long long*>(counters), partials, y);
    } else if constexpr (EPI == kEpiStore && MB == 1) {
        // one activation row (MB == 1 is M == 1 in every plan): every wave reports for itself
        splitk_exchange_store_per_wave(psum[0], N, ct, kt, ktiles, ct, partials, counters, y);
    } else if constexpr (EPI == kEpiStore) {
        splitk_exchange_store<MB>(psum, m0, M, N, ct, kt, ktiles, blockIdx.z * coltiles + ct, partials, counters, y,
                                  &s_prev);
    } else if constexpr (EPI == kEpiResidual) {
        static_assert(MB == 1, "the residual epilogue serves one activation row");
        // every wave of 64 columns finishes for itself (splitk_exchange_sum_per_wave) and leaves the sum of
        // squares of its quarter of the tile: no barrier, no wave waits for another
        float sum;
        if (!splitk_exchange_sum_per_wave(psum[0], &sum, N, ct, kt, ktiles, ct, partials, counters)) return;
        const int col = ct * kTileCols + tid;
        float r = 0.0f;
        if (col < N) {
            const float o = bf16_to_f32(f32_to_bf16(sum));  // the projection's output is a bf16 tensor
            const uint16_t rbits = f32_to_bf16(bf16_to_f32(resid_pre) + o);
            store_result(res.out + col, rbits);
            r = bf16_to_f32(rbits);
        }
        const float q = wave_sum(r * r);
        if (lane == 0) store_result(res.sumsq + ct * (kTileCols / kWave) + tid / kWave, q);
    } else {
        static_assert(MB == 1, "the rotary epilogue serves one activation row");
        // A column tile is two heads of 128 (the host admits whole tiles only).  The finished row is rounded
        // to bf16 as a separate GEMV would store it; lane i of the finishing wave holds elements i and i + 64
        // of its head, the layout of the per-head routine.
        if (ktiles == 1) {
            // no exchange: the two waves of a head meet in LDS
            __shared__ uint16_t s_row[kTileCols];
            if (tid < kTileCols) s_row[tid] = f32_to_bf16(psum[0]);
            __syncthreads();
            if (tid < kTileCols && (tid & 64) == 0) {
                const int local = tid >> 7;
                const int head = ct * (kTileCols / kHeadDim) + local;
                qk_norm_rope_head_at<true>(s_row[local * kHeadDim + lane], s_row[local * kHeadDim + lane + 64], head, lane,
                                           rope, rope_pos, rope_gain_a, rope_gain_b, rope_sin, rope_cos);
            }
        } else {
            // the last of the head's waves over all K tiles finishes the head: no barrier, no LDS
            float lo, hi;
            if (!splitk_exchange_sum_per_head(psum[0], &lo, &hi, N, ct, kt, ktiles, partials, counters)) return;
            const int head = ct * (kTileCols / kHeadDim) + (tid >> 7);
            qk_norm_rope_head_at<true>(f32_to_bf16(lo), f32_to_bf16(hi), head, lane, rope, rope_pos, rope_gain_a,
                                       rope_gain_b, rope_sin, rope_cos);
        }
    }
}

template <int WAVES, int RT, int MB, int PRO = kProNone, int EPI = kEpiStore>
inline void launch_awq_gemv(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                            const int32_t* qzeros, uint16_t* y, float* partials, uint32_t* counters,
                            int M, int K, int N, int group, int coltiles, int ktiles, int mtiles,
                            hipStream_t stream, const FusedInput& fi = FusedInput{},
                            const RopeTarget& rope = RopeTarget{}, const ResidualTarget& res = ResidualTarget{}) {
    dim3 grid(coltiles, ktiles, mtiles);
    dim3 block(WAVES * kWave, 1, 1);
    int group_shift = -1;  // log2(group) where it is a power of two
    for (int sh = 0; sh < 31; sh++) {
        if ((1 << sh) == group) group_shift = sh;
    }
    hipLaunchKernelGGL((awq_gemv_kernel<WAVES, RT, MB, PRO, EPI>), grid, block, 0, stream, x,
                       reinterpret_cast<const uint32_t*>(qweight), scales,
                       reinterpret_cast<const uint32_t*>(qzeros), y, partials, counters, M, K, N,
                       group, group_shift, coltiles, ktiles, fi, rope, res);
}

}  // namespace kx

#endif  // KX_AWQ_GEMV_KERNEL_H
