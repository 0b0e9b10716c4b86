// Supporting kernels of a Qwen3-style decode step (batch 1) for gfx950: RMSNorm (optionally fused
// with the residual add), per-head QK-norm + RoPE + KV-cache append, GQA flash-decoding (split over
// the context, merged by log-sum-exp), SwiGLU, residual add, embedding row copy and argmax.
// All of them are HBM- or latency-bound byte movers; arithmetic is fp32, storage bf16.
//
// The reference reserves layer slots for these operators (LayerRMSNorm, LayerRope, LayerMHA,
// LayerSwiGLU, LayerAdd, LayerEmbedding: kuiper/include/op/layer.h:8-20) and names their scratch
// buffers (model::ModelBufferType, kuiper/include/base/base.h:12-31) but implements none of them
// except the fp32 add (kuiper/source/op/kernel/cuda/add_kernel.cu:4-12).
#include "kx_attn_merge.h"
#include "kx_common.h"
#include "kx_rope.h"

#include <math.h>

namespace kx {
namespace {

__device__ __forceinline__ void unpack8(const uint4& raw, float (&out)[8]) {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        out[2 * i] = __uint_as_float(w[i] << 16);
        out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}

__device__ __forceinline__ uint4 pack8(const float (&v)[8]) {
    uint4 out;
    out.x = f32x2_to_bf16x2(v[0], v[1]);
    out.y = f32x2_to_bf16x2(v[2], v[3]);
    out.z = f32x2_to_bf16x2(v[4], v[5]);
    out.w = f32x2_to_bf16x2(v[6], v[7]);
    return out;
}

// ------------------------------------------------------------------------------------------------
// RMSNorm over rows of n elements: y = w * bf16(x * rsqrt(mean(x^2) + eps)), the rounding points of
// the usual Qwen3 formulation (normalise in fp32, round, then scale by the bf16 gain).
// With `delta` the row is first updated in place, x <- bf16(x + delta) (the residual add), and the
// norm is taken of the updated row.  One workgroup per row, eight elements per thread per pass.
// ------------------------------------------------------------------------------------------------
constexpr int kNormThreads = 512;

template <bool ADD>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_kernel(uint16_t* __restrict__ x,
                                                               const uint16_t* __restrict__ delta,
                                                               const uint16_t* __restrict__ w,
                                                               uint16_t* __restrict__ y, int n, float eps) {
    __shared__ float red[kNormThreads / kWave];
    const size_t row = blockIdx.x;
    uint16_t* xr = x + row * n;
    const uint16_t* dr = ADD ? delta + row * n : nullptr;
    uint16_t* yr = y + row * n;
    const int chunks = n >> 3;

    // first pass: (update and) sum of squares; a row of up to 4096 elements stays in registers
    float keep[8];
    bool have = false;
    float ss = 0.0f;
    for (int c = threadIdx.x; c < chunks; c += kNormThreads) {
        float v[8];
        unpack8(reinterpret_cast<const uint4*>(xr)[c], v);
        if (ADD) {
            float d[8];
            unpack8(reinterpret_cast<const uint4*>(dr)[c], d);
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = bf16_to_f32(f32_to_bf16(v[i] + d[i]));
            reinterpret_cast<uint4*>(xr)[c] = pack8(v);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) ss += v[i] * v[i];
        if (c == static_cast<int>(threadIdx.x)) {
#pragma unroll
            for (int i = 0; i < 8; i++) keep[i] = v[i];
            have = true;
        }
    }
    ss = wave_sum(ss);
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = ss;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < kNormThreads / kWave; i++) total += red[i];
    const float inv = 1.0f / sqrtf(total / static_cast<float>(n) + eps);

    for (int c = threadIdx.x; c < chunks; c += kNormThreads) {
        float v[8], g[8];
        if (have && c == static_cast<int>(threadIdx.x)) {
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = keep[i];
        } else {
            unpack8(reinterpret_cast<const uint4*>(xr)[c], v);
        }
        unpack8(reinterpret_cast<const uint4*>(w)[c], g);
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = g[i] * bf16_to_f32(f32_to_bf16(v[i] * inv));
        reinterpret_cast<uint4*>(yr)[c] = pack8(v);
    }
}

// ------------------------------------------------------------------------------------------------
// Per-head RMSNorm (gain over head_dim = 128) of the query and key heads, rotary embedding at
// position `pos` in the rotate-half convention, and the KV-cache append:
//   qkv  bf16 [ (n_q + 2 n_kv) * 128 ]   = q heads | k heads | v heads, the output of a fused QKV GEMV
//   q_out bf16 [n_q * 128]
//   k_cache, v_cache bf16 [max_pos][n_kv][128]; row `pos` is written
// One wave per head; lane i holds elements i and i + 64, the two partners of the rotation.
//   out[i]      = x[i] * cos(pos f_i) - x[i+64] * sin(pos f_i)
//   out[i + 64] = x[i+64] * cos(pos f_i) + x[i] * sin(pos f_i),     f_i = theta^(-i/64)
// ------------------------------------------------------------------------------------------------
// Several sequences decoded together: blockIdx.y is the sequence; row b of qkv and q_out, position pos[b] and
// the cache pair that starts b * cache_stride elements into k_cache / v_cache belong to sequence b.
__global__ __launch_bounds__(256) void qk_norm_rope_kernel(const uint16_t* __restrict__ qkv, RopeTarget t,
                                                           size_t cache_stride) {
    const int head = blockIdx.x * 4 + threadIdx.x / kWave;  // 0 .. n_q + 2 n_kv - 1
    const int lane = threadIdx.x % kWave;
    const int heads = t.n_q + 2 * t.n_kv;
    if (head >= heads) return;
    const size_t seq = blockIdx.y;
    t.q_out += seq * t.n_q * kHeadDim;
    t.k_cache += seq * cache_stride;
    t.v_cache += seq * cache_stride;
    t.pos += seq;
    const uint16_t* src = qkv + (seq * heads + head) * kHeadDim;
    qk_norm_rope_head(src[lane], src[lane + 64], head, lane, t);
}

// ------------------------------------------------------------------------------------------------
// GQA flash-decoding, head_dim 128, one query position.
// Stage 1: a workgroup takes one KV head and one chunk of CHUNK (64 or 128) cache positions and serves the
// G = n_q / n_kv query heads of that KV head together, so every K and V row is read once.  The
// scores q . K come from the matrix cores, sixteen positions per tile; they go to LDS, softmax
// statistics are taken per head over the chunk, then the V rows (loaded sixteen lanes per position,
// one contiguous 256-byte row each, and staged in LDS) are accumulated with the chunk-local weights,
// again on the matrix cores.  Output per (KV head, chunk): for each of the
// G heads the unnormalised 128-vector, the chunk maximum and the chunk sum of exponentials.
// Stage 2: one wave per query head merges the chunks by log-sum-exp and writes bf16.
// ------------------------------------------------------------------------------------------------
constexpr int kAttnThreads = 256;
constexpr int kMaxGroup = 16;  // query heads per KV head: the rows of one MFMA tile

template <int CHUNK>
__global__ __launch_bounds__(kAttnThreads) void attn_decode_stage1(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
    float* __restrict__ part_out, float* __restrict__ part_ml, int n_kv, int G, const int32_t* __restrict__ pos_ptr,
    int nchunks, int max_positions, float scale, size_t cache_stride) {
    // Scores, then softmax weights, per head; rows padded so that the sixteen-byte reads of the
    // second pass (one row per lane) do not all start on the same bank.
    __shared__ __attribute__((aligned(16))) float s_score[kMaxGroup][CHUNK + 4];
    // The chunk's V rows, row-major, two dwords of padding per row: the second pass reads a dword (two
    // neighbouring dims) of eight positions per lane, and with 66 dwords per row the four blocks of eight
    // positions that a read instruction touches fall on different banks.
    constexpr int kVRow = kHeadDim / 2 + 2;
    __shared__ __attribute__((aligned(8))) uint32_t s_v[CHUNK][kVRow];

    const int kvh = blockIdx.y;
    const int chunk = blockIdx.x;
    const int p0 = chunk * CHUNK;
    const int tid = threadIdx.x;
    {
        // several sequences decoded together: blockIdx.z is the sequence, with its own query row, cache pair
        // (cache_stride elements apart), position and slice of the two result arrays
        const size_t seq = blockIdx.z;
        const size_t heads = static_cast<size_t>(n_kv) * G;
        q += seq * heads * kHeadDim;
        k_cache += seq * cache_stride;
        v_cache += seq * cache_stride;
        pos_ptr += seq;
        part_out += seq * nchunks * heads * kHeadDim;
        part_ml += seq * nchunks * heads * 2;
    }
    const int sub = tid % 16;    // which eight dims of the row
    const int slot = tid / 16;   // position slot inside the workgroup: 16 slots

    // Every K and V row of this lane is requested before anything is consumed, and the addresses do
    // not depend on *pos: any row below max_positions exists, rows past the context are masked once
    // the position has arrived.  The chunk then costs one memory round trip.
    const size_t row_stride = static_cast<size_t>(n_kv) * kHeadDim;  // elements between positions
    constexpr int ITERS = CHUNK / 16;
    // Scores on the matrix cores: per tile of sixteen positions, D[head][position] = sum over the 128
    // dims in four steps of 32, A = the query heads (row = head, zero rows past G), B = the K rows
    // (column = position).  Lane (c = lane % 16, b = lane / 16) supplies dims 32 s + 8 b .. + 7 of head
    // c and of position c, sixteen contiguous bytes each.  A wave takes TPW of the chunk's tiles.
    constexpr int kWaves = kAttnThreads / kWave;
    constexpr int TPW = ITERS / kWaves;  // position tiles per wave: 1 (chunks of 64) or 2 (128)
    static_assert(ITERS % kWaves == 0, "whole tiles per wave");
    const int wave = tid / kWave;
    const int mc = (tid % kWave) % 16;
    const int mb = (tid % kWave) / 16;
    // The query heads are requested first: loads return in order, and the scores need q and K but
    // not V, so q must not queue behind the V rows.
    u32x4 qraw[4];
    const int q_head = mc < G ? mc : G - 1;  // clamped: rows past G are zeroed below
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        qraw[ks] = *reinterpret_cast<const u32x4*>(q + (static_cast<size_t>(kvh) * G + q_head) * kHeadDim + 32 * ks + 8 * mb);
    }
    u32x4 kraw[TPW][4], vraw[ITERS];
#pragma unroll
    for (int t = 0; t < TPW; t++) {
        const int p = p0 + (wave * TPW + t) * 16 + mc;
        const int pc = p < max_positions ? p : max_positions - 1;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            kraw[t][ks] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(
                k_cache + pc * row_stride + static_cast<size_t>(kvh) * kHeadDim + 32 * ks + 8 * mb));
        }
    }
#pragma unroll
    for (int it = 0; it < ITERS; it++) {
        const int p = p0 + it * 16 + slot;
        const int pc = p < max_positions ? p : max_positions - 1;
        vraw[it] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(
            v_cache + pc * row_stride + static_cast<size_t>(kvh) * kHeadDim + 8 * sub));
    }
    const int ctx = pos_ptr[0] + 1;  // positions 0 .. pos are valid (pos was appended just before)
    __builtin_amdgcn_sched_barrier(0);

    const bool one_sequence = gridDim.z == 1;  // write-through results for the one-row step only (store_result)
    float* out_base = part_out + (static_cast<size_t>(kvh) * nchunks + chunk) * G * kHeadDim;
    float* ml_base = part_ml + (static_cast<size_t>(kvh) * nchunks + chunk) * G * 2;
    // No early exit for a chunk past the end of the context: a branch on *pos ahead of the loads
    // lets the compiler sink every K and V load below it, and the chunk then costs the round trip
    // for *pos and the round trip for the rows one after the other.  Such a chunk runs through with
    // everything masked and reports max = -inf, sum = 0.

#if defined(KX_ABLATE) && KX_ABLATE == 4
    {  // profiling build: loads only - fold what arrived into one word and leave
        uint32_t f = static_cast<uint32_t>(ctx);
#pragma unroll
        for (int ks = 0; ks < 4; ks++) f ^= qraw[ks].x ^ qraw[ks].w;
#pragma unroll
        for (int t = 0; t < TPW; t++)
#pragma unroll
            for (int ks = 0; ks < 4; ks++) f ^= kraw[t][ks].x ^ kraw[t][ks].y ^ kraw[t][ks].z ^ kraw[t][ks].w;
#pragma unroll
        for (int it = 0; it < ITERS; it++) f ^= vraw[it].x ^ vraw[it].y ^ vraw[it].z ^ vraw[it].w;
        if (f == 0x9E3779B9u) out_base[tid] = 1.0f;
        return;
    }
#endif
    // pass 1: scores, in units of log 2 (the exponentials below and in the merge are the hardware's exp2)
    const float scale2 = scale * 1.44269504088896341f;
    const bool q_live = mc < G;
#pragma unroll
    for (int t = 0; t < TPW; t++) {
        f32x4v d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const bf16x8 a_op = as_bf16x8(q_live ? qraw[ks].x : 0u, q_live ? qraw[ks].y : 0u,
                                          q_live ? qraw[ks].z : 0u, q_live ? qraw[ks].w : 0u);
            const bf16x8 b_op = as_bf16x8(kraw[t][ks].x, kraw[t][ks].y, kraw[t][ks].z, kraw[t][ks].w);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_op, b_op, d, 0, 0, 0);
        }
        // the lane holds heads 4 mb .. 4 mb + 3 of position mc of the tile
        const int pl = (wave * TPW + t) * 16 + mc;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            // rows past G exist in s_score and nobody reads them: no test, no branch around the store
            s_score[4 * mb + v][pl] = (p0 + pl < ctx) ? d[v] * scale2 : -INFINITY;
        }
    }
    // LDS only: the V rows stay in flight, and the statistics below run while they arrive (a full
    // __syncthreads() would make the scores wait for every V row)
    lds_barrier();

    // softmax statistics per head over the chunk; wave w serves heads w, w + 4, ...
    for (int g = tid / kWave; g < G; g += kAttnThreads / kWave) {
        const int lane = tid % kWave;
        constexpr int PER_LANE = CHUNK / kWave;
        float sc[PER_LANE];
        float m = -INFINITY;
#pragma unroll
        for (int u = 0; u < PER_LANE; u++) {
            sc[u] = s_score[g][lane + u * kWave];
            m = fmaxf(m, sc[u]);
        }
        m = wave_max(m);
        const float shift = m == -INFINITY ? 0.0f : m;  // a chunk with no valid position: all weights 0
        float l = 0.0f;
#pragma unroll
        for (int u = 0; u < PER_LANE; u++) {
            sc[u] = __builtin_amdgcn_exp2f(sc[u] - shift);
            l += sc[u];
            s_score[g][lane + u * kWave] = sc[u];
        }
        l = wave_sum(l);
        if (lane == 0) {
            if (one_sequence) {
                store_result(ml_base + 2 * g, m);
                store_result(ml_base + 2 * g + 1, l);
            } else {
                ml_base[2 * g] = m;
                ml_base[2 * g + 1] = l;
            }
        }
    }

    // pass 2, in two halves of the chunk: the V rows of a half go to LDS (rows past the context carry weight 0,
    // their arbitrary contents are zeroed so that a stray NaN or infinity cannot leak through 0 * x), a barrier,
    // and the half's weighted sum of V rows on the matrix cores, D[head][dim] = sum over the half's positions in
    // steps of 32, A = the softmax weights (row = head), B = the V rows (column = dim).  The first half is summed
    // while the rows of the second are still arriving (loads return in order), so that only the second half's
    // chain stands behind the last byte.
    // Lane (mc, mb) supplies positions 32 s + 8 mb .. + 7 of head mc and of one dim.  A wave takes 32 dims as two
    // tiles, the even dims and the odd ones, so that one dword read per position feeds both.  The weights are
    // fp32 and the operands bf16: a weight enters as its bf16 rounding plus the bf16 rounding of what that left
    // over, two MFMAs per step (error 2^-17 relative instead of 2^-9).
#if defined(KX_ABLATE) && KX_ABLATE == 5
    {  // profiling build: scores and statistics, then wait for the V rows and leave
        uint32_t f = 0;
#pragma unroll
        for (int it = 0; it < ITERS; it++) f ^= vraw[it].x ^ vraw[it].y ^ vraw[it].z ^ vraw[it].w;
        if (f == 0x9E3779B9u) out_base[tid] = s_score[0][tid % CHUNK];
        return;
    }
#endif
    constexpr int KSTEPS = CHUNK / 32;
    static_assert(ITERS % 2 == 0 && KSTEPS % 2 == 0, "two halves of whole steps");
    f32x4v dacc[2];
    dacc[0] = dacc[1] = f32x4v{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int half = 0; half < 2; half++) {
#pragma unroll
        for (int i = 0; i < ITERS / 2; i++) {
            const int it = half * (ITERS / 2) + i;
            const int pl = it * 16 + slot;
            const bool live = p0 + pl < ctx;
            u32x2* dst = reinterpret_cast<u32x2*>(&s_v[pl][4 * sub]);
            dst[0] = u32x2{live ? vraw[it].x : 0u, live ? vraw[it].y : 0u};
            dst[1] = u32x2{live ? vraw[it].z : 0u, live ? vraw[it].w : 0u};
        }
        lds_barrier();  // the first one also publishes the weights
#pragma unroll
        for (int k = 0; k < KSTEPS / 2; k++) {
            const int ks = half * (KSTEPS / 2) + k;
            const float4* prow = reinterpret_cast<const float4*>(&s_score[q_head][32 * ks + 8 * mb]);
            const float4 pa = prow[0];
            const float4 pb = prow[1];
            const float pw[8] = {pa.x, pa.y, pa.z, pa.w, pb.x, pb.y, pb.z, pb.w};
            uint32_t hi[4], lo[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float w0 = q_live ? pw[2 * j] : 0.0f;
                const float w1 = q_live ? pw[2 * j + 1] : 0.0f;
                hi[j] = f32x2_to_bf16x2(w0, w1);
                lo[j] = f32x2_to_bf16x2(w0 - __uint_as_float(hi[j] << 16), w1 - __uint_as_float(hi[j] & 0xffff0000u));
            }
            const bf16x8 a_hi = as_bf16x8(hi[0], hi[1], hi[2], hi[3]);
            const bf16x8 a_lo = as_bf16x8(lo[0], lo[1], lo[2], lo[3]);
            // dims 32 wave + 2 mc (low half of the dword) and + 1 (high half) of eight positions
            uint32_t vd[8];
#pragma unroll
            for (int j = 0; j < 8; j++) vd[j] = s_v[32 * ks + 8 * mb + j][16 * wave + mc];
            uint32_t even[4], odd[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                even[j] = __builtin_amdgcn_perm(vd[2 * j + 1], vd[2 * j], 0x05040100u);  // low halves of two positions
                odd[j] = __builtin_amdgcn_perm(vd[2 * j + 1], vd[2 * j], 0x07060302u);   // high halves
            }
            const bf16x8 b_even = as_bf16x8(even[0], even[1], even[2], even[3]);
            const bf16x8 b_odd = as_bf16x8(odd[0], odd[1], odd[2], odd[3]);
            dacc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, b_even, dacc[0], 0, 0, 0);
            dacc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, b_odd, dacc[1], 0, 0, 0);
            dacc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, b_even, dacc[0], 0, 0, 0);
            dacc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, b_odd, dacc[1], 0, 0, 0);
        }
    }
    // The lane holds heads 4 mb .. 4 mb + 3 of dims 32 wave + 2 mc and + 1: one eight-byte store per head.
    // One test on the kind of store and one on the lane's heads around all four stores: inside the loop they
    // had become two branches per store.  (A lane's four heads are all live or all past G when G is a multiple
    // of four; other groupings take the per-head test.)
#if defined(KX_ABLATE) && KX_ABLATE == 6
    // profiling build: everything but the stores of the weighted sums
    if (dacc[0][0] + dacc[1][1] + dacc[0][2] + dacc[1][3] != 12345.678f) return;
#endif
    const bool all_four = 4 * mb + 3 < G;
    const int dim0 = 32 * wave + 2 * mc;
    if (one_sequence && all_four) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const u32x2 pair = {__float_as_uint(dacc[0][v]), __float_as_uint(dacc[1][v])};
            unsigned long long bits;
            __builtin_memcpy(&bits, &pair, 8);
            store_result(reinterpret_cast<unsigned long long*>(out_base + (4 * mb + v) * kHeadDim + dim0), bits);
        }
    } else {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int head = 4 * mb + v;
            if (all_four || head < G) {
                *reinterpret_cast<float2*>(out_base + head * kHeadDim + dim0) = make_float2(dacc[0][v], dacc[1][v]);
            }
        }
    }
}

constexpr int kMergeThreads = kHeadDim * kMergeParts;

__global__ __launch_bounds__(kMergeThreads) void attn_decode_stage2(const float* __restrict__ part_out,
                                                                    const float* __restrict__ part_ml,
                                                                    uint16_t* __restrict__ out, int G, int nchunks,
                                                                    int per_part) {
    // rescaling factors exp(m_c - m), per_part slots for each of the four chunk subsets (attn_factor_slot);
    // slots of chunks that do not exist hold 0
    extern __shared__ __attribute__((aligned(16))) float s_factor[];
    __shared__ float s_norm;
    __shared__ float s_part[kMergeParts][kHeadDim];
    const int head = blockIdx.x;  // query head
    const int kvh = head / G;
    const int g = head % G;
    const int tid = threadIdx.x;
    {
        const size_t seq = blockIdx.y;  // several sequences decoded together
        const size_t heads = gridDim.x;
        part_out += seq * nchunks * heads * kHeadDim;
        part_ml += seq * nchunks * heads * 2;
        out += seq * heads * kHeadDim;
    }
    // thread (part, d) sums dimension d over the chunks c = part, part + 4, ...
    const int d = tid % kHeadDim;
    const int part = tid / kHeadDim;
    const float* po = part_out + (static_cast<size_t>(kvh) * nchunks * G + g) * kHeadDim + d;
    const size_t cstride = static_cast<size_t>(G) * kHeadDim;
    // The partial sums do not depend on the rescaling factors: the first kMergeFront chunks of this
    // thread are requested before the statistics, so the kernel costs one trip to memory for both
    // instead of one for the statistics and one per batch of eight chunks after it.  Clamped
    // addresses, masked use: straight-line loads.
    constexpr int kMergeFront = 32;  // chunks per thread in that first flight: 128 chunks of the context
    float front[kMergeFront];
#pragma unroll
    for (int u = 0; u < kMergeFront; u++) {
        const int c = part + u * kMergeParts;
        front[u] = po[(c < nchunks ? c : nchunks - 1) * cstride];
    }
    __builtin_amdgcn_sched_barrier(0);
    if (tid < kWave) {
        const MergeStats<kMergeLanesLong> st =
            attn_merge_load<kMergeLanesLong>(part_ml + static_cast<size_t>(kvh) * nchunks * G * 2, g, G, nchunks, tid);
        const float l = attn_merge_finish<kMergeLanesLong>(st, s_factor, per_part, tid);
        if (tid == 0) s_norm = l;
    }
    __syncthreads();

    // The thread's factors lie side by side and absent chunks carry factor 0: straight-line code.  (A test
    // on the chunk count per step had been compiled to a branch and an LDS read with a full wait per chunk.)
    float acc = 0.0f;
    const float* fpart = s_factor + part * per_part;  // per_part >= kMergeFront, a multiple of four
    static_assert(kMergeFront % 4 == 0, "the factors are read four at a time");
#pragma unroll
    for (int u4 = 0; u4 < kMergeFront / 4; u4++) {
        const float4 f = reinterpret_cast<const float4*>(fpart)[u4];
        acc = attn_merge_step(acc, front[4 * u4], f.x);
        acc = attn_merge_step(acc, front[4 * u4 + 1], f.y);
        acc = attn_merge_step(acc, front[4 * u4 + 2], f.z);
        acc = attn_merge_step(acc, front[4 * u4 + 3], f.w);
    }
    // what a longer context leaves, in batches as before; the order of the additions is unchanged
    for (int c0 = part + kMergeFront * kMergeParts; c0 < nchunks; c0 += kMergeBatch * kMergeParts) {
        float v[kMergeBatch];
#pragma unroll
        for (int u = 0; u < kMergeBatch; u++) {
            const int c = c0 + u * kMergeParts;
            // straight-line loads: a chunk past the end reads the last one, an empty chunk whatever its
            // slot holds; attn_merge_step and the guard below leave both out of the sum
            v[u] = po[(c < nchunks ? c : nchunks - 1) * cstride];
        }
#pragma unroll
        for (int u = 0; u < kMergeBatch; u++) {
            const int c = c0 + u * kMergeParts;
            if (c < nchunks) acc = attn_merge_step(acc, v[u], s_factor[attn_factor_slot(c, per_part)]);
        }
    }
    s_part[part][d] = acc;
    __syncthreads();
    if (part == 0) {
        // no position to attend to (*pos < 0): zeros rather than 0 / 0
        const float total = (s_part[0][d] + s_part[1][d]) + (s_part[2][d] + s_part[3][d]);
        out[static_cast<size_t>(head) * kHeadDim + d] = f32_to_bf16(s_norm > 0.0f ? total / s_norm : 0.0f);
    }
}

// ------------------------------------------------------------------------------------------------
// Elementwise: SwiGLU, residual add.  Eight elements per thread, grid-stride.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void swiglu_kernel(const uint16_t* __restrict__ gate,
                                                     const uint16_t* __restrict__ up,
                                                     uint16_t* __restrict__ out, int chunks) {
    for (int c = blockIdx.x * blockDim.x + threadIdx.x; c < chunks; c += gridDim.x * blockDim.x) {
        float g[8], u[8];
        unpack8(reinterpret_cast<const uint4*>(gate)[c], g);
        unpack8(reinterpret_cast<const uint4*>(up)[c], u);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            // silu(g) is a bf16 tensor before it meets `up` in the usual formulation
            const float act = silu_rounded_to_bf16(g[i]);
            g[i] = act * u[i];
        }
        reinterpret_cast<uint4*>(out)[c] = pack8(g);
    }
}

__global__ __launch_bounds__(256) void add_bf16_kernel(const uint16_t* __restrict__ a,
                                                       const uint16_t* __restrict__ b,
                                                       uint16_t* __restrict__ out, int chunks) {
    for (int c = blockIdx.x * blockDim.x + threadIdx.x; c < chunks; c += gridDim.x * blockDim.x) {
        float x[8], y[8];
        unpack8(reinterpret_cast<const uint4*>(a)[c], x);
        unpack8(reinterpret_cast<const uint4*>(b)[c], y);
#pragma unroll
        for (int i = 0; i < 8; i++) x[i] += y[i];
        reinterpret_cast<uint4*>(out)[c] = pack8(x);
    }
}

__global__ __launch_bounds__(256) void embedding_kernel(const uint16_t* __restrict__ table,
                                                        const int32_t* __restrict__ token_ptr,
                                                        uint16_t* __restrict__ out, int chunks, int vocab) {
    int token = token_ptr[blockIdx.y];  // blockIdx.y: which of the tokens looked up together
    token = token < 0 ? 0 : (token >= vocab ? vocab - 1 : token);
    const uint4* row = reinterpret_cast<const uint4*>(table + static_cast<size_t>(token) * chunks * 8);
    uint4* dst = reinterpret_cast<uint4*>(out) + static_cast<size_t>(blockIdx.y) * chunks;
    for (int c = blockIdx.x * blockDim.x + threadIdx.x; c < chunks; c += gridDim.x * blockDim.x) {
        dst[c] = row[c];
    }
}

// argmax over n bf16 values, first index on ties, NaN ignored; one workgroup.
// Two passes, because one compute unit's vector ALUs are what bounds it: the first takes the maximum
// alone (one v_max per element instead of two compares and two selects), the second looks for the
// first index that holds it, and only in the threads whose own maximum is the overall one.
constexpr int kArgmaxThreads = 1024;
__global__ __launch_bounds__(kArgmaxThreads) void argmax_kernel(const uint16_t* __restrict__ x, int n,
                                                               int32_t* __restrict__ out, size_t ld) {
    x += blockIdx.x * ld;  // one workgroup per row
    out += blockIdx.x;
    constexpr int kWaves = kArgmaxThreads / kWave;
    __shared__ float s_val[kWaves];
    __shared__ int s_idx[kWaves];
    const int tid = threadIdx.x;
    const bool wide = (reinterpret_cast<uintptr_t>(x) % 16) == 0;
    const int chunks = wide ? n / 8 : 0;
    const uint4* xv = reinterpret_cast<const uint4*>(x);

    // First sweep: twenty 16-byte loads per thread, all in flight together and kept in registers —
    // the 151 936 logits of the Qwen3 vocabulary are one sweep, i.e. one trip to memory, and the
    // search for the index below needs no second one.  Clamped addresses: straight-line loads; a
    // piece past the end re-reads the last one, which cannot change a maximum.
    float mine = -INFINITY;  // fmaxf drops a NaN operand
    constexpr int kHeld = 20;
    uint4 held[kHeld];
#pragma unroll
    for (int u = 0; u < kHeld; u++) held[u] = make_uint4(0u, 0u, 0u, 0u);
    if (chunks > 0) {  // nothing is read from an input without a whole 16-byte piece
#pragma unroll
        for (int u = 0; u < kHeld; u++) {
            const int c = tid + u * kArgmaxThreads;
            held[u] = xv[c < chunks ? c : chunks - 1];
        }
#pragma unroll
        for (int u = 0; u < kHeld; u++) {
            float v[8];
            unpack8(held[u], v);
#pragma unroll
            for (int i = 0; i < 8; i++) mine = fmaxf(mine, v[i]);
        }
    }
    // longer inputs: further sweeps of eight loads
    constexpr int kInFlight = 8;
    for (int c0 = tid + kHeld * kArgmaxThreads; c0 < chunks; c0 += kInFlight * kArgmaxThreads) {
        uint4 raw[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; u++) {
            const int c = c0 + u * kArgmaxThreads;
            raw[u] = xv[c < chunks ? c : chunks - 1];
        }
#pragma unroll
        for (int u = 0; u < kInFlight; u++) {
            float v[8];
            unpack8(raw[u], v);
#pragma unroll
            for (int i = 0; i < 8; i++) mine = fmaxf(mine, v[i]);
        }
    }
    for (int i = 8 * chunks + tid; i < n; i += kArgmaxThreads) mine = fmaxf(mine, bf16_to_f32(x[i]));
    const float wave_best = wave_max(mine);
    if (tid % kWave == 0) s_val[tid / kWave] = wave_best;
    __syncthreads();
    float best = s_val[0];
#pragma unroll
    for (int w = 1; w < kWaves; w++) best = fmaxf(best, s_val[w]);

    int first = 0x7fffffff;
    if (mine == best) {  // few threads: they walk their own elements again (-0 and +0 are one value)
#pragma unroll
        for (int u = kHeld - 1; u >= 0; u--) {  // the held pieces, from registers
            const int c = tid + u * kArgmaxThreads;
            float v[8];
            unpack8(held[u], v);
#pragma unroll
            for (int i = 7; i >= 0; i--) {
                if (c < chunks && v[i] == best) first = 8 * c + i;  // descending walk: the last hit is the first index
            }
        }
        if (first == 0x7fffffff) {  // not among the held pieces: the later sweeps, re-read
            for (int c = tid + kHeld * kArgmaxThreads; c < chunks; c += kArgmaxThreads) {
                float v[8];
                unpack8(xv[c], v);
#pragma unroll
                for (int i = 7; i >= 0; i--) {
                    if (v[i] == best && 8 * c + i < first) first = 8 * c + i;
                }
            }
            for (int i = 8 * chunks + tid; i < n; i += kArgmaxThreads) {
                if (bf16_to_f32(x[i]) == best && i < first) first = i;
            }
        }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const int other = __shfl_xor(first, off, kWave);
        first = other < first ? other : first;
    }
    if (tid % kWave == 0) s_idx[tid / kWave] = first;
    __syncthreads();
    if (tid == 0) {
#pragma unroll
        for (int w = 0; w < kWaves; w++) first = s_idx[w] < first ? s_idx[w] : first;
        out[0] = first == 0x7fffffff ? 0 : first;  // nothing but NaN: index 0
    }
}

inline bool aligned16(const void* p) {
    return (reinterpret_cast<uintptr_t>(p) % 16) == 0;
}

}  // namespace
}  // namespace kx

extern "C" int kx_rmsnorm_bf16(const uint16_t* x, const uint16_t* gain, uint16_t* y, int32_t rows, int32_t n,
                               float eps, void* stream) {
    if (!x || !gain || !y) return KX_ERR_NULL_POINTER;
    if (rows < 1 || n < 8 || (n % 8) != 0) return KX_ERR_BAD_SHAPE;
    if (!kx::aligned16(x) || !kx::aligned16(gain) || !kx::aligned16(y)) return KX_ERR_ALIGNMENT;
    hipLaunchKernelGGL((kx::rmsnorm_kernel<false>), dim3(rows), dim3(kx::kNormThreads), 0, kx::as_stream(stream),
                       const_cast<uint16_t*>(x), static_cast<const uint16_t*>(nullptr), gain, y, n, eps);
    return kx::launch_status();
}

extern "C" int kx_add_rmsnorm_bf16(uint16_t* x_inout, const uint16_t* delta, const uint16_t* gain, uint16_t* y,
                                   int32_t rows, int32_t n, float eps, void* stream) {
    if (!x_inout || !delta || !gain || !y) return KX_ERR_NULL_POINTER;
    if (rows < 1 || n < 8 || (n % 8) != 0) return KX_ERR_BAD_SHAPE;
    if (!kx::aligned16(x_inout) || !kx::aligned16(delta) || !kx::aligned16(gain) || !kx::aligned16(y)) {
        return KX_ERR_ALIGNMENT;
    }
    hipLaunchKernelGGL((kx::rmsnorm_kernel<true>), dim3(rows), dim3(kx::kNormThreads), 0, kx::as_stream(stream),
                       x_inout, delta, gain, y, n, eps);
    return kx::launch_status();
}

extern "C" int kx_qk_norm_rope_bf16(const uint16_t* qkv, const uint16_t* q_gain, const uint16_t* k_gain,
                                    uint16_t* q_out, uint16_t* k_cache, uint16_t* v_cache, int32_t n_q_heads,
                                    int32_t n_kv_heads, int32_t head_dim, const int32_t* pos,
                                    int32_t cache_positions, float rope_theta, float eps, void* stream) {
    if (!qkv || !q_gain || !k_gain || !q_out || !k_cache || !v_cache || !pos) return KX_ERR_NULL_POINTER;
    if (head_dim != kx::kHeadDim || n_q_heads < 1 || n_kv_heads < 1 || cache_positions < 1 || !(rope_theta > 1.0f)) {
        return KX_ERR_BAD_SHAPE;
    }
    return kx_qk_norm_rope_batch_bf16(qkv, q_gain, k_gain, q_out, k_cache, v_cache, 0, n_q_heads, n_kv_heads, head_dim,
                                      pos, cache_positions, rope_theta, eps, 1, stream);
}

extern "C" int kx_qk_norm_rope_batch_bf16(const uint16_t* qkv, const uint16_t* q_gain, const uint16_t* k_gain,
                                          uint16_t* q_out, uint16_t* k_cache, uint16_t* v_cache, size_t cache_stride,
                                          int32_t n_q_heads, int32_t n_kv_heads, int32_t head_dim, const int32_t* pos,
                                          int32_t cache_positions, float rope_theta, float eps, int32_t batch,
                                          void* stream) {
    if (!qkv || !q_gain || !k_gain || !q_out || !k_cache || !v_cache || !pos) return KX_ERR_NULL_POINTER;
    if (head_dim != kx::kHeadDim || n_q_heads < 1 || n_kv_heads < 1 || cache_positions < 1 || !(rope_theta > 1.0f) ||
        batch < 1 || batch > KX_MAX_BATCH) {
        return KX_ERR_BAD_SHAPE;
    }
    // consecutive caches must not overlap
    if (batch > 1 && cache_stride < static_cast<size_t>(cache_positions) * n_kv_heads * kx::kHeadDim) return KX_ERR_BAD_SHAPE;
    const int heads = n_q_heads + 2 * n_kv_heads;
    kx::RopeTarget t{q_gain, k_gain, q_out, k_cache, v_cache, pos, cache_positions, n_q_heads, n_kv_heads,
                     log2f(rope_theta), eps};
    hipLaunchKernelGGL(kx::qk_norm_rope_kernel, dim3((heads + 3) / 4, batch), dim3(256), 0, kx::as_stream(stream), qkv,
                       t, cache_stride);
    return kx::launch_status();
}

extern "C" size_t kx_attn_decode_workspace_bytes(int32_t n_q_heads, int32_t head_dim, int32_t max_positions) {
    if (n_q_heads < 1 || head_dim != kx::kHeadDim || max_positions < 1) return 0;
    const size_t nchunks = static_cast<size_t>(kx::attn_chunks_of(max_positions));
    return nchunks * n_q_heads * (kx::kHeadDim + 2) * sizeof(float);
}

namespace {
// Shared by the two attention entry points: checks, then the first stage and (with `out`) the merge.
int attn_decode(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache, uint16_t* out,
                int32_t n_q_heads, int32_t n_kv_heads, int32_t head_dim, const int32_t* pos, int32_t max_positions,
                void* workspace, size_t workspace_bytes, void* stream, int32_t batch = 1, size_t cache_stride = 0) {
    if (!q || !k_cache || !v_cache || !pos || !workspace) return KX_ERR_NULL_POINTER;
    if (head_dim != kx::kHeadDim || n_q_heads < 1 || n_kv_heads < 1 || (n_q_heads % n_kv_heads) != 0 ||
        max_positions < 1 || batch < 1 || batch > KX_MAX_BATCH) {
        return KX_ERR_BAD_SHAPE;
    }
    const int G = n_q_heads / n_kv_heads;
    if (G > kx::kMaxGroup) return KX_ERR_BAD_SHAPE;
    if (batch > 1 && ((cache_stride % 8) != 0 ||
                      cache_stride < static_cast<size_t>(max_positions) * n_kv_heads * kx::kHeadDim)) {
        return KX_ERR_BAD_SHAPE;  // every cache 16-byte aligned, none inside another
    }
    if (workspace_bytes < batch * kx_attn_decode_workspace_bytes(n_q_heads, head_dim, max_positions)) return KX_ERR_WORKSPACE;
    if (!kx::aligned16(q) || !kx::aligned16(k_cache) || !kx::aligned16(v_cache) || !kx::aligned16(workspace)) {
        return KX_ERR_ALIGNMENT;
    }
    // From four sequences on the first stage takes chunks of 128 positions whatever the cache length (measured at
    // context 4096: + 0.6 % tokens/s at four sequences, + 0.9 % at eight, + 3.7 % at sixteen; one sequence loses
    // 0.35 us per layer that way): half as many workgroups and per-chunk results for the same bytes.  Only where
    // the merge follows here: the o projection's merge prologue counts on the chunking of one sequence.
    const bool long_chunks = kx::attn_chunk_for(max_positions) == kx::kAttnChunkLong || (out && batch >= 4);
    const int chunk = long_chunks ? kx::kAttnChunkLong : kx::kAttnChunkShort;
    const int nchunks = (max_positions + chunk - 1) / chunk;  // at most attn_chunks_of(max_positions): the workspace fits
    if (nchunks > kx::kMergeLanesLong * kx::kWave) return KX_ERR_BAD_SHAPE;  // 65536 positions
    // the unnormalised vectors of every sequence first, then the statistics of every sequence
    float* part_out = static_cast<float*>(workspace);
    float* part_ml = part_out + static_cast<size_t>(batch) * nchunks * n_q_heads * kx::kHeadDim;
    const float scale = 1.0f / sqrtf(static_cast<float>(kx::kHeadDim));
    hipStream_t s = kx::as_stream(stream);
    dim3 grid1(nchunks, n_kv_heads, batch);
    if (long_chunks) {
        hipLaunchKernelGGL((kx::attn_decode_stage1<kx::kAttnChunkLong>), grid1, dim3(kx::kAttnThreads), 0, s, q, k_cache,
                           v_cache, part_out, part_ml, n_kv_heads, G, pos, nchunks, max_positions, scale, cache_stride);
    } else {
        hipLaunchKernelGGL((kx::attn_decode_stage1<kx::kAttnChunkShort>), grid1, dim3(kx::kAttnThreads), 0, s, q, k_cache,
                           v_cache, part_out, part_ml, n_kv_heads, G, pos, nchunks, max_positions, scale, cache_stride);
    }
    if (out) {
        // slots per chunk subset: the straight-line first flight of the merge covers 32, longer contexts more
        int per_part = (nchunks + kx::kMergeParts - 1) / kx::kMergeParts;
        if (per_part < 32) per_part = 32;
        per_part = (per_part + 3) / 4 * 4;
        hipLaunchKernelGGL(kx::attn_decode_stage2, dim3(n_q_heads, batch), dim3(kx::kMergeThreads),
                           kx::kMergeParts * per_part * sizeof(float), s, part_out, part_ml, out, G, nchunks, per_part);
    }
    return kx::launch_status();
}
}  // namespace

extern "C" int kx_attn_decode_bf16(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                                   uint16_t* out, int32_t n_q_heads, int32_t n_kv_heads, int32_t head_dim,
                                   const int32_t* pos, int32_t max_positions, void* workspace,
                                   size_t workspace_bytes, void* stream) {
    if (!out) return KX_ERR_NULL_POINTER;
    return attn_decode(q, k_cache, v_cache, out, n_q_heads, n_kv_heads, head_dim, pos, max_positions, workspace,
                       workspace_bytes, stream);
}

extern "C" int kx_attn_decode_batch_bf16(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                                         size_t cache_stride, uint16_t* out, int32_t n_q_heads, int32_t n_kv_heads,
                                         int32_t head_dim, const int32_t* pos, int32_t max_positions, void* workspace,
                                         size_t workspace_bytes, int32_t batch, void* stream) {
    if (!out) return KX_ERR_NULL_POINTER;
    return attn_decode(q, k_cache, v_cache, out, n_q_heads, n_kv_heads, head_dim, pos, max_positions, workspace,
                       workspace_bytes, stream, batch, cache_stride);
}

extern "C" int kx_attn_decode_partial_bf16(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                                           int32_t n_q_heads, int32_t n_kv_heads, int32_t head_dim,
                                           const int32_t* pos, int32_t max_positions, void* workspace,
                                           size_t workspace_bytes, void* stream) {
    return attn_decode(q, k_cache, v_cache, nullptr, n_q_heads, n_kv_heads, head_dim, pos, max_positions, workspace,
                       workspace_bytes, stream);
}

extern "C" int kx_swiglu_bf16(const uint16_t* gate, const uint16_t* up, uint16_t* out, int32_t n, void* stream) {
    if (!gate || !up || !out) return KX_ERR_NULL_POINTER;
    if (n < 8 || (n % 8) != 0) return KX_ERR_BAD_SHAPE;
    if (!kx::aligned16(gate) || !kx::aligned16(up) || !kx::aligned16(out)) return KX_ERR_ALIGNMENT;
    const int chunks = n / 8;
    int blocks = (chunks + 255) / 256;
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(kx::swiglu_kernel, dim3(blocks), dim3(256), 0, kx::as_stream(stream), gate, up, out, chunks);
    return kx::launch_status();
}

extern "C" int kx_add_bf16(const uint16_t* a, const uint16_t* b, uint16_t* out, int32_t n, void* stream) {
    if (!a || !b || !out) return KX_ERR_NULL_POINTER;
    if (n < 8 || (n % 8) != 0) return KX_ERR_BAD_SHAPE;
    if (!kx::aligned16(a) || !kx::aligned16(b) || !kx::aligned16(out)) return KX_ERR_ALIGNMENT;
    const int chunks = n / 8;
    int blocks = (chunks + 255) / 256;
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(kx::add_bf16_kernel, dim3(blocks), dim3(256), 0, kx::as_stream(stream), a, b, out, chunks);
    return kx::launch_status();
}

extern "C" int kx_embedding_bf16(const uint16_t* table, const int32_t* token, uint16_t* out, int32_t vocab,
                                 int32_t dim, void* stream) {
    if (!table || !token || !out) return KX_ERR_NULL_POINTER;
    if (vocab < 1 || dim < 8 || (dim % 8) != 0) return KX_ERR_BAD_SHAPE;
    if (!kx::aligned16(table) || !kx::aligned16(out)) return KX_ERR_ALIGNMENT;
    return kx_embedding_rows_bf16(table, token, out, vocab, dim, 1, stream);
}

extern "C" int kx_embedding_rows_bf16(const uint16_t* table, const int32_t* tokens, uint16_t* out, int32_t vocab,
                                      int32_t dim, int32_t rows, void* stream) {
    if (!table || !tokens || !out) return KX_ERR_NULL_POINTER;
    if (vocab < 1 || dim < 8 || (dim % 8) != 0 || rows < 1 || rows > 65535) return KX_ERR_BAD_SHAPE;
    if (!kx::aligned16(table) || !kx::aligned16(out)) return KX_ERR_ALIGNMENT;
    const int chunks = dim / 8;
    hipLaunchKernelGGL(kx::embedding_kernel, dim3((chunks + 255) / 256, rows), dim3(256), 0, kx::as_stream(stream),
                       table, tokens, out, chunks, vocab);
    return kx::launch_status();
}

extern "C" int kx_argmax_bf16(const uint16_t* x, int32_t n, int32_t* out_index, void* stream) {
    return kx_argmax_rows_bf16(x, n, n, out_index, 1, stream);
}

extern "C" int kx_argmax_rows_bf16(const uint16_t* x, int32_t n, int32_t ld, int32_t* out_index, int32_t rows,
                                   void* stream) {
    if (!x || !out_index) return KX_ERR_NULL_POINTER;
    if (n < 1 || rows < 1 || (rows > 1 && ld < n)) return KX_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(kx::argmax_kernel, dim3(rows), dim3(kx::kArgmaxThreads), 0, kx::as_stream(stream), x, n,
                       out_index, static_cast<size_t>(ld));
    return kx::launch_status();
}
