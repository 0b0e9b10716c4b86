// A measured alternative to the one-shot GEMV kernels, kept selectable (KX_POLICY_STREAM of the internal entry
// point) so that the comparison can be repeated: resident workgroups that walk a K loop.
//
//   y[m,n] = sum_k x[m,k] * (q[k,n] - z[k/G,n]) * s[k/G,n]                      (gfx950, matrix cores, M <= 4)
//
// The arithmetic is that of kx_awq_gemv_mfma_kernel.h.  The matrix is cut into units of 32 rows of K x 256
// columns (one MFMA step of one wave, 4 KiB of packed weights), numbered column tile by column tile, and the
// G <= 256 workgroups - one per compute unit, eight waves - each take one contiguous run of U/G units
// ("stream-K"): every compute unit streams the same number of bytes whatever the shape, and a run touches at
// most two column tiles (the host keeps G >= number of column tiles).  Inside a workgroup the eight waves split
// each of the (one or two) segments of the run into eight contiguous chunks, and a wave walks its chunk with the
// loads of the next unit in flight while it works on the current one: weights (eight 8-byte buffer loads per
// lane), the scales and zero words of the unit's quantisation group, and the activations.  The row offset of a
// unit travels in a scalar register (buffer loads take one), so a load costs no vector ALU work.
//
// Raw sums are turned into scaled sums whenever a wave leaves a quantisation group:
//   tot[n] += s[g,n] * (acc[n] - (128 + z[g,n]) * sum_k x[k])
// At the end of a segment a wave leaves its totals in LDS; when the run is done the two halves of the
// workgroup (threads 0..255 and 256..511) add the eight waves' totals of segment 0 and 1, one column per
// thread, and meet the other workgroups of their column tile in the split-K workspace as in the one-shot
// kernels (partial sums written through, arrival counter, last arriver adds in slot order).
//
// What it measured against the one-shot kernels (us per launch, M = 1, cold weights): it loses wherever a
// launch is short - 4096->4096 7.9 against 5.7, 4096->12288 10.4 against 8.5, 4096->24576 14.0 against 13.0 -
// and wins only on the tallest shape, 25600->5120 17.9 against 18.6; 5120->51200 is 29.8 against 29.3.  Two
// things hold it back: with one unit in flight per wave a wave is bound by the latency of its own loads (a
// deeper ring costs a compute unit's vector-memory issue slots on padding units - it takes one vector-memory
// instruction per ~12 ns whatever its width - and was slower at every depth tried), and the second wave of
// each SIMD, which the instruction arbiter serves after the first, finishes a quarter later than the first
// (alternating s_setprio between the two changed nothing).  The one-shot kernels stay the default.
#ifndef KX_AWQ_GEMV_STREAM_KERNEL_H
#define KX_AWQ_GEMV_STREAM_KERNEL_H

#include "kx_awq_gemv_mfma_kernel.h"
#include "kx_common.h"
#include "kx_splitk_exchange.h"

namespace kx {

constexpr int kMaxStreamGrid = 256;  // one workgroup per compute unit of an MI355X

// Everything the kernel needs arrives in one batch of kernel arguments; what would take an integer
// division on the device (how units fall onto workgroups and column tiles) the host works out once.
struct StreamArgs {
    const uint16_t* x;
    const uint32_t* qweight;
    const uint16_t* scales;
    const uint32_t* qzeros;
    uint16_t* y;
    float* partials;
    uint32_t* counters;
    int M, K, N;
    int group_shift;
    int S;          // 32-row steps per column tile, K / 32
    int U;          // units in all: column tiles * S (below 2^24)
    int G;          // workgroups
    int lo, rem;    // workgroup w takes lo + (w < rem) units starting at w * lo + min(w, rem)
    uint32_t mS, mlo, mlo1;   // n / d == (n * m) >> sh for 0 <= n < 2^24, d = S, lo, lo + 1
    int shS, shlo, shlo1;
};

__device__ __forceinline__ int div_magic(int n, uint32_t m, int sh) {
    return static_cast<int>((static_cast<unsigned long long>(static_cast<uint32_t>(n)) * m) >> sh);
}

__device__ __forceinline__ int stream_first_unit(int w, const StreamArgs& a) {
    return w * a.lo + (w < a.rem ? w : a.rem);
}

// the workgroup whose run holds unit t
__device__ __forceinline__ int stream_owner_of(int t, const StreamArgs& a) {
    const int big = a.rem * (a.lo + 1);  // units held by the workgroups that take lo + 1
    return t < big ? div_magic(t, a.mlo1, a.shlo1) : a.rem + div_magic(t - big, a.mlo, a.shlo);
}

template <int WAVES, int VR, int P>
__global__ __launch_bounds__(WAVES * kWave, 1) void awq_gemv_stream_kernel(StreamArgs a) {
    static_assert(WAVES == 4 || WAVES == 8, "one or two waves per SIMD");
    static_assert(VR == 1 || VR == 2 || VR == 4, "activation rows a lane's first D rows can hold");
    static_assert(P >= 2 && P <= 6, "units in flight per wave");
    constexpr int THREADS = WAVES * kWave;
    constexpr int HALVES = THREADS / kTileCols;  // groups of 256 threads: each finishes one segment at a time
    extern __shared__ __attribute__((aligned(16))) float red[];  // [2 segments][WAVES][VR][256]
    __shared__ uint32_t s_prev[2];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int lane = tid % kWave;
    const int c = lane % 16;  // word pair c of the tile, MFMA column c
    const int b = lane / 16;  // k block inside a step, D row block
    const int S = a.S, N = a.N, M = a.M;
    const int nw = N >> 3;
    const int spg_mask = (1 << (a.group_shift - 5)) - 1;  // steps per quantisation group - 1
    // The run of this workgroup: units [u0, u0 + len), at most two segments (tile ct0 from step begin0 on,
    // then the head of tile ct0 + 1).  Scalars and selects rather than small arrays: an array indexed by
    // the segment would live in scratch.
    const int wg = blockIdx.x;
    const int u0 = stream_first_unit(wg, a);
    const int len = a.lo + (wg < a.rem ? 1 : 0);
    const int ct0 = div_magic(u0, a.mS, a.shS);
    const int begin0 = u0 - ct0 * S;
    const int room = S - begin0;
    const int len0 = len < room ? len : room;
    const int len1 = len - len0;
    const int nseg = len1 > 0 ? 2 : 1;
    // this wave's chunk of each segment: [cb, cb + cn), padded to a multiple of P slots
    constexpr int LOGW = WAVES == 8 ? 3 : 2;
    const int lo0 = (wave * len0) >> LOGW, hi0 = ((wave + 1) * len0) >> LOGW;
    const int lo1 = (wave * len1) >> LOGW, hi1 = ((wave + 1) * len1) >> LOGW;
    const int cb0 = begin0 + lo0, cn0 = hi0 - lo0;
    const int cb1 = lo1, cn1 = hi1 - lo1;
    const int pad0 = (cn0 + P - 1) / P * P, pad1 = (cn1 + P - 1) / P * P;
    const int slots = pad0 + pad1;

    // Buffer resources: raw buffers of the tensors' own sizes (the host keeps each below 2 GiB).
    constexpr int kRsrcFlags = 0x00020000;
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(a.qweight), 0, static_cast<int>(static_cast<uint32_t>(static_cast<size_t>(a.K) * nw * 4)), kRsrcFlags);
    const int groups = a.K >> a.group_shift;
    const __amdgpu_buffer_rsrc_t rs_s = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(a.scales), 0, static_cast<int>(static_cast<uint32_t>(static_cast<size_t>(groups) * N * 2)), kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs_z = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(a.qzeros), 0, static_cast<int>(static_cast<uint32_t>(static_cast<size_t>(groups) * nw * 4)), kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(a.x), 0, static_cast<int>(static_cast<uint32_t>(static_cast<size_t>(M) * a.K * 2)), kRsrcFlags);
    constexpr int kNonTemporal = 2;
    // lane offsets in bytes; the unit's offset is added as a scalar
    const int vo_w = (8 * b * nw + 2 * c) * 4;
    const int vo_s = 16 * c * 2;
    const int vo_z = 2 * c * 4;
    const int vo_x = ((c < M ? c : M - 1) * a.K + 8 * b) * 2;
    const bool x_live = c < M;

    // ring of P units
    uint32_t w[P][8][2];
    u32x4 sc[P][2];
    u32x2 zw[P];
    u32x4 xa[P];

    // Slot i of the wave's sequence: the padded chunk of segment 0, then that of segment 1.  Loads for slot
    // i + P - 1 are issued while slot i is worked on.
    auto fetch = [&](const int st, const int slot) {
        const bool second = slot >= pad0;
        const int pos = slot - (second ? pad0 : 0);
        const bool real = slot < slots && pos < (second ? cn1 : cn0);
        const int step = (second ? cb1 : cb0) + pos;
        const int ct = ct0 + (second ? 1 : 0);
        // A slot that only pads the sequence reads the first bytes of each tensor, every lane the same
        // address: one cache line that is always at hand.  (Pointing such a slot past the end of the buffer
        // also returns without data, but measured 0.7 us per slot.)
        const int g = (step * kStepRows) >> a.group_shift;
        const int so_w = real ? (step * kStepRows * nw + ct * 32) * 4 : 0;
        const int so_s = real ? (g * N + ct * kTileCols) * 2 : 0;
        const int so_z = real ? (g * nw + ct * 32) * 4 : 0;
        const int so_x = real ? step * kStepRows * 2 : 0;
        const int rstride = real ? nw * 4 : 0;
        const int lw = real ? vo_w : 0;
        const int ls = real ? vo_s : 0;
        const int lz = real ? vo_z : 0;
        const int lx = real ? vo_x : 0;
#pragma unroll
        for (int r = 0; r < 8; r++) {
            const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rs_w, lw, so_w + r * rstride, kNonTemporal);
            w[st][r][0] = v.x;
            w[st][r][1] = v.y;
        }
        sc[st][0] = __builtin_amdgcn_raw_buffer_load_b128(rs_s, ls, so_s, 0);
        sc[st][1] = __builtin_amdgcn_raw_buffer_load_b128(rs_s, ls + 16, so_s, 0);
        zw[st] = __builtin_amdgcn_raw_buffer_load_b64(rs_z, lz, so_z, 0);
        xa[st] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, lx, so_x, 0);
    };

    const bf16x8 ones = as_bf16x8(0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u);
    const f32x4v zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    const uint32_t magic = opaque_bf16_128_pair();
    f32x4v xs = zero4;
    f32x4v acc[2][8];
    float tot[2][8][VR];
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int p = 0; p < 8; p++) {
            acc[h][p] = zero4;
#pragma unroll
            for (int v = 0; v < VR; v++) tot[h][p][v] = 0.0f;
        }
    }

    auto compute = [&](const int st, bool leaves_group) {
        const bf16x8 a_op = as_bf16x8(x_live ? xa[st].x : 0u, x_live ? xa[st].y : 0u, x_live ? xa[st].z : 0u,
                                      x_live ? xa[st].w : 0u);
        xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_op, ones, xs, 0, 0, 0);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint32_t bop[8][4];  // [nibble p][row pair]
#pragma unroll
            for (int rp = 0; rp < 4; rp++) {
                const uint32_t wa = w[st][2 * rp][h];
                const uint32_t wb = w[st][2 * rp + 1][h];
                const uint32_t lo = __builtin_amdgcn_perm(wb, wa, 0x05040100u);  // nibbles 0..3 of both rows
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
                    a_op, as_bf16x8(bop[p][0], bop[p][1], bop[p][2], bop[p][3]), acc[h][p], 0, 0, 0);
            }
        }
        if (leaves_group) {  // wave-uniform
            const uint32_t sw[8] = {sc[st][0].x, sc[st][0].y, sc[st][0].z, sc[st][0].w,
                                    sc[st][1].x, sc[st][1].y, sc[st][1].z, sc[st][1].w};
            const uint32_t zws[2] = {zw[st].x, zw[st].y};
#pragma unroll
            for (int h = 0; h < 2; h++) {
#pragma unroll
                for (int p = 0; p < 8; p++) {
                    const int j = 8 * h + order_of(p);  // column inside the lane's sixteen
                    const uint16_t sbits = static_cast<uint16_t>((j & 1) ? (sw[j >> 1] >> 16) : (sw[j >> 1] & 0xffffu));
                    const float s = f16_bits_to_f32(sbits);
                    const float zoff = 128.0f + static_cast<float>((zws[h] >> (4 * p)) & 0xFu);
#pragma unroll
                    for (int v = 0; v < VR; v++) {
                        tot[h][p][v] = __builtin_fmaf(s, __builtin_fmaf(-zoff, xs[v], acc[h][p][v]), tot[h][p][v]);
                    }
                    acc[h][p] = zero4;
                }
            }
            xs = zero4;
        }
    };

    // the wave's totals of a segment go to LDS (D rows 0..3 live in lanes 0..15), zeros if it had no unit
    auto leave_segment = [&](const int seg) {
        if (b == 0) {
#pragma unroll
            for (int v = 0; v < VR; v++) {
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    f32x4* dst = reinterpret_cast<f32x4*>(&red[((seg * WAVES + wave) * VR + v) * kTileCols + 16 * c + 8 * h]);
                    dst[0] = f32x4{tot[h][nibble_of(0)][v], tot[h][nibble_of(1)][v], tot[h][nibble_of(2)][v],
                                   tot[h][nibble_of(3)][v]};
                    dst[1] = f32x4{tot[h][nibble_of(4)][v], tot[h][nibble_of(5)][v], tot[h][nibble_of(6)][v],
                                   tot[h][nibble_of(7)][v]};
                }
            }
        }
#pragma unroll
        for (int h = 0; h < 2; h++) {
#pragma unroll
            for (int p = 0; p < 8; p++) {
#pragma unroll
                for (int v = 0; v < VR; v++) tot[h][p][v] = 0.0f;
            }
        }
    };

    // ---- the run ----
#pragma unroll
    for (int j = 0; j < P - 1; j++) fetch(j, j);
    __builtin_amdgcn_sched_barrier(0);  // the first loads leave before the rest of the set-up is worked through
    if (nseg == 2 && pad0 == 0) leave_segment(0);

#pragma unroll 1
    for (int i = 0; i < slots; i += P) {
#pragma unroll
        for (int j = 0; j < P; j++) {
            fetch((j + P - 1) % P, i + j + P - 1);
            const int slot = i + j;
            const bool second = slot >= pad0;
            const int pos = slot - (second ? pad0 : 0);
            const int cn = second ? cn1 : cn0;
            if (pos < cn) {  // wave-uniform
                const int step = (second ? cb1 : cb0) + pos;
                compute(j, pos == cn - 1 || ((step + 1) & spg_mask) == 0);
            }
        }
        if (nseg == 2 && i + P == pad0) leave_segment(0);
    }
    leave_segment(nseg - 1);
    __syncthreads();

    // ---- the end of the run: each group of 256 threads finishes a segment, one column per thread ----
    const int half = __builtin_amdgcn_readfirstlane(tid / kTileCols);
    const int t = tid % kTileCols;
    constexpr int ROUNDS = 2 / HALVES;  // segments a group of 256 threads may have to finish
    const size_t tstride = static_cast<size_t>(M) * N;
    float psum[ROUNDS][VR];
    int ord[ROUNDS], count[ROUNDS];
#pragma unroll
    for (int rd = 0; rd < ROUNDS; rd++) {
        const int seg = half + rd * HALVES;
        const bool have = seg < nseg;
        const int segc = have ? seg : 0;
        const int ct = ct0 + segc;
#pragma unroll
        for (int v = 0; v < VR; v++) {
            float sum = 0.0f;
#pragma unroll
            for (int u = 0; u < WAVES; u++) sum += red[((segc * WAVES + u) * VR + v) * kTileCols + t];
            psum[rd][v] = sum;
        }
        const int first_w = stream_owner_of(ct * S, a);
        const int last_w = stream_owner_of(ct * S + S - 1, a);
        count[rd] = have ? last_w - first_w + 1 : 1;
        ord[rd] = wg - first_w;
        if (count[rd] > 1) {
            const int col = ct * kTileCols + t;
#pragma unroll
            for (int v = 0; v < VR; v++) {
                if (v < M) store_agent(a.partials + static_cast<size_t>(ord[rd]) * tstride + static_cast<size_t>(v) * N + col, psum[rd][v]);
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (t == 0) {
#pragma unroll
        for (int rd = 0; rd < ROUNDS; rd++) {
            const int seg = half + rd * HALVES;
            if (seg < 2) {
                uint32_t* counter = a.counters + static_cast<size_t>(ct0 + seg) * kCounterStride;
                s_prev[seg] = count[rd] > 1 ? __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int rd = 0; rd < ROUNDS; rd++) {
        const int seg = half + rd * HALVES;
        if (seg >= nseg) continue;
        const int ct = ct0 + seg;
        const int col = ct * kTileCols + t;
        float sum[VR];
        if (count[rd] == 1) {
#pragma unroll
            for (int v = 0; v < VR; v++) sum[v] = psum[rd][v];
        } else {
            if (s_prev[seg] != static_cast<uint32_t>(count[rd] - 1)) continue;
            // last to arrive for this tile: add the partials in slot order
#pragma unroll
            for (int v = 0; v < VR; v++) sum[v] = 0.0f;
            constexpr int TB = 8;
            for (int t0 = 0; t0 < count[rd]; t0 += TB) {
                float got[VR][TB];
#pragma unroll
                for (int v = 0; v < VR; v++) {
#pragma unroll
                    for (int u = 0; u < TB; u++) {
                        const int slot = t0 + u;
                        const int sc_ = slot < count[rd] ? slot : count[rd] - 1;
                        const int vc = v < M ? v : M - 1;
                        const float g = load_agent(a.partials + static_cast<size_t>(sc_) * tstride + static_cast<size_t>(vc) * N + col);
                        got[v][u] = (slot < count[rd] && v < M) ? g : 0.0f;
                    }
                }
#pragma unroll
                for (int v = 0; v < VR; v++) {
#pragma unroll
                    for (int u = 0; u < TB; u++) sum[v] += got[v][u];
                }
            }
            if (t == 0) {
                __hip_atomic_store(a.counters + static_cast<size_t>(ct) * kCounterStride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
#pragma unroll
        for (int v = 0; v < VR; v++) {
            if (v < M) a.y[static_cast<size_t>(v) * N + col] = f32_to_bf16(sum[v]);
        }
    }
}

// LDS the kernel asks for at launch
inline size_t stream_lds_bytes(int waves, int vr) {
    return static_cast<size_t>(2) * waves * vr * kTileCols * sizeof(float);
}

}  // namespace kx

#endif  // KX_AWQ_GEMV_STREAM_KERNEL_H
