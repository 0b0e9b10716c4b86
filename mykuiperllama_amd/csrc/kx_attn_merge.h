// Log-sum-exp merge of the per-chunk results of the flash-decoding kernel, shared by the stand-alone
// merge kernel and by the prologue of the o-projection GEMV so that both produce the same bits.
//
// Per KV head the first stage leaves, for every chunk c of the context and each of its G query heads:
//   part_out[kvh][c][g][0..127]   the unnormalised weighted sum of V rows, relative to the chunk maximum
//   part_ml [kvh][c][g][0..1]     the chunk maximum m_c of the scores in units of log 2 (score * log2 e) and the
//                                 chunk sum of exponentials l_c (0: empty chunk)
// The merged head is  sum_c part_out[c] * f_c / sum_c l_c * f_c  with  f_c = 2^(m_c - max_c m_c), the hardware's
// exponential (v_exp_f32) like the first stage's.
#ifndef KX_ATTN_MERGE_H
#define KX_ATTN_MERGE_H

#include <math.h>

#include "kx_common.h"

namespace kx {

// Cache positions per chunk of the first stage: 64 for caches of up to 5120 positions (more, smaller
// workgroups: the first stage is a chain of latencies), 128 beyond, which keeps the number of chunks
// of a cache of up to 10240 positions within what the o projection can merge in its prologue.
constexpr int kAttnChunkShort = 64;
constexpr int kAttnChunkLong = 128;
constexpr int kAttnShortLimit = 80 * kAttnChunkShort;
__host__ __device__ constexpr int attn_chunk_for(int max_positions) {
    return max_positions <= kAttnShortLimit ? kAttnChunkShort : kAttnChunkLong;
}
__host__ __device__ constexpr int attn_chunks_of(int max_positions) {
    return (max_positions + attn_chunk_for(max_positions) - 1) / attn_chunk_for(max_positions);
}
constexpr int kMergeParts = 4;      // a dimension is summed over the chunks c = p, p + 4, ... for p = 0..3 side by side
constexpr int kMergeBatch = 8;      // loads in flight per thread in the stand-alone merge
constexpr int kMergeLanesLong = 8;  // chunks per lane the stand-alone merge provides for: 512 chunks

// Chunk statistics of head (kvh, g) as one wave holds them: lane i has chunks i, i + 64, ...
// (PER_LANE of them; chunks past nchunks read as empty).  Loading and finishing are separate so
// that a caller can put other loads between the two.
template <int PER_LANE>
struct MergeStats {
    float m[PER_LANE];
    float l[PER_LANE];
};

template <int PER_LANE>
__device__ __forceinline__ MergeStats<PER_LANE> attn_merge_load(const float* __restrict__ ml, int g, int G,
                                                               int nchunks, int lane) {
    MergeStats<PER_LANE> st;
#pragma unroll
    for (int u = 0; u < PER_LANE; u++) {
        const int c = lane + u * kWave;
        const int cc = c < nchunks ? c : nchunks - 1;  // clamped: the loads are straight-line code
        const float mc = ml[(static_cast<size_t>(cc) * G + g) * 2];
        const float lc = ml[(static_cast<size_t>(cc) * G + g) * 2 + 1];
        st.m[u] = c < nchunks ? mc : -INFINITY;
        st.l[u] = c < nchunks ? lc : 0.0f;
    }
    return st;
}

// Where the factor of chunk c lies in a table of `per_part` entries for each of the kMergeParts chunk
// subsets: a thread that sums the chunks c = p, p + 4, ... finds its factors side by side.
__device__ __forceinline__ int attn_factor_slot(int c, int per_part) {
    return (c % kMergeParts) * per_part + c / kMergeParts;
}

// Writes the factor of every chunk below kMergeParts * per_part to its slot of s_factor (0 for a chunk
// past nchunks or without a valid position, so that the sums over the table need no test on the chunk
// count) and returns the normaliser, the same value in every lane.  The result does not depend on
// PER_LANE (absent chunks are neutral).
template <int PER_LANE>
__device__ __forceinline__ float attn_merge_finish(const MergeStats<PER_LANE>& st, float* s_factor, int per_part,
                                                   int lane) {
    float m = -INFINITY;
#pragma unroll
    for (int u = 0; u < PER_LANE; u++) m = fmaxf(m, st.m[u]);
    m = wave_max(m);
    float l = 0.0f;
#pragma unroll
    for (int u = 0; u < PER_LANE; u++) {
        const int c = lane + u * kWave;
        const float f = st.l[u] > 0.0f ? __builtin_amdgcn_exp2f(st.m[u] - m) : 0.0f;  // chunks past the context have l == 0
        if (c < kMergeParts * per_part) s_factor[attn_factor_slot(c, per_part)] = f;
        l += st.l[u] * f;
    }
    return wave_sum(l);
}

// acc <- acc + v * f for a chunk that holds something; the partial sums of an empty chunk were never
// written and are not looked at
__device__ __forceinline__ float attn_merge_step(float acc, float v, float f) {
    return __builtin_fmaf(f > 0.0f ? v : 0.0f, f, acc);
}

}  // namespace kx

#endif  // KX_ATTN_MERGE_H
