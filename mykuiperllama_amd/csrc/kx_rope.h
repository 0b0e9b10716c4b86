// Per-head RMSNorm + rotary embedding + KV-cache append for one head of a fused q|k|v row, as one
// wave executes it.  Shared by the stand-alone kernel and by the epilogue of the q/k/v GEMV so that
// both produce the same bits.
#ifndef KX_ROPE_H
#define KX_ROPE_H

#include <math.h>

#include "kx_common.h"

namespace kx {

constexpr int kHeadDim = 128;

struct RopeTarget {
    const uint16_t* q_gain;   // bf16 [128]
    const uint16_t* k_gain;   // bf16 [128]
    uint16_t* q_out;          // bf16 [n_q * 128]
    uint16_t* k_cache;        // bf16 [cache_positions][n_kv][128]; row *pos is written
    uint16_t* v_cache;
    const int32_t* pos;       // device scalar
    int cache_positions;      // rows the caches hold: a position outside 0 .. cache_positions-1 writes no row
    int n_q;
    int n_kv;
    float log2_theta;
    float eps;
};

// Called by the 64 lanes of one wave; lane i brings elements i and i + 64 of head `head`
// (0 .. n_q + 2 n_kv - 1, query heads first, then key heads, then value heads) as bf16 bits.
//   out[i]      = x[i] * cos(pos f_i) - x[i+64] * sin(pos f_i)
//   out[i + 64] = x[i+64] * cos(pos f_i) + x[i] * sin(pos f_i),     f_i = theta^(-i/64)
// where x is the head after RMSNorm (rounded to bf16, as a bf16 norm layer returns it).
// `pos`, `gain_a` and `gain_b` are *t.pos and elements lane and lane + 64 of the head's gain (q_gain for a
// query head, k_gain for a key head, unused for a value head): a caller that knows early which head
// a wave will serve loads them ahead of time.
__device__ __forceinline__ void qk_norm_rope_head_with(uint16_t a_bits, uint16_t b_bits, int head, int lane,
                                                       const RopeTarget& t, int pos, uint16_t gain_a,
                                                       uint16_t gain_b) {
    const bool row_ok = static_cast<unsigned>(pos) < static_cast<unsigned>(t.cache_positions);
    if (head >= t.n_q + t.n_kv) {  // value head: straight into the cache
        if (row_ok) {
            uint16_t* dst = t.v_cache + (static_cast<size_t>(pos) * t.n_kv + (head - t.n_q - t.n_kv)) * kHeadDim;
            dst[lane] = a_bits;
            dst[lane + 64] = b_bits;
        }
        return;
    }
    const float a = bf16_to_f32(a_bits);
    const float b = bf16_to_f32(b_bits);
    const bool is_q = head < t.n_q;
    const float ss = wave_sum(a * a + b * b);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(kHeadDim) + t.eps);
    const float na = bf16_to_f32(gain_a) * bf16_to_f32(f32_to_bf16(a * inv));
    const float nb = bf16_to_f32(gain_b) * bf16_to_f32(f32_to_bf16(b * inv));
    // the norm output is a bf16 tensor in the usual formulation; the rotation starts from that
    const float xa = bf16_to_f32(f32_to_bf16(na));
    const float xb = bf16_to_f32(f32_to_bf16(nb));
    const float freq = exp2f(-t.log2_theta * static_cast<float>(lane) / 64.0f);
    float s, c;
    sincosf(static_cast<float>(pos) * freq, &s, &c);
    const float oa = xa * c - xb * s;
    const float ob = xb * c + xa * s;
    uint16_t* dst = is_q ? t.q_out + static_cast<size_t>(head) * kHeadDim
                         : t.k_cache + (static_cast<size_t>(pos) * t.n_kv + (head - t.n_q)) * kHeadDim;
    if (is_q || row_ok) {
        dst[lane] = f32_to_bf16(oa);
        dst[lane + 64] = f32_to_bf16(ob);
    }
}

// The same with the three operands loaded here.
__device__ __forceinline__ void qk_norm_rope_head(uint16_t a_bits, uint16_t b_bits, int head, int lane,
                                                  const RopeTarget& t) {
    const uint16_t* gain = head < t.n_q ? t.q_gain : t.k_gain;  // a value head reads k_gain and ignores it
    qk_norm_rope_head_with(a_bits, b_bits, head, lane, t, t.pos[0], gain[lane], gain[lane + 64]);
}

}  // namespace kx

#endif  // KX_ROPE_H
