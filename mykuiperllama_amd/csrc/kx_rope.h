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

// sin and cos of a rotary angle, 0 <= x < 2^17 (positions below 65536 times a frequency of at most 1).
// The library routine carries a large-argument path that keeps a table in private memory, which makes
// every kernel that calls it a kernel with scratch memory; the angles here never need it.  Reduction to
// [-pi/4, pi/4] in double (x - k pi/2 with k = rint(x 2/pi): two operations, exact enough for any k below
// 2^17), then the classic single-precision minimax polynomials (error below 1 ulp of the result) and the
// quadrant.
__device__ __forceinline__ void rope_sincos(float x, float* s_out, float* c_out) {
    const float kf = rintf(x * 0.63661977236758134f);
    const float r = static_cast<float>(__builtin_fma(static_cast<double>(-kf), 1.5707963267948966, static_cast<double>(x)));
    const float z = r * r;
    const float sp = r + r * z * (-1.6666654611e-1f + z * (8.3321608736e-3f + z * -1.9515295891e-4f));
    const float cp = 1.0f - 0.5f * z + z * z * (4.166664568298827e-2f + z * (-1.388731625493765e-3f + z * 2.443315711809948e-5f));
    const int q = static_cast<int>(kf) & 3;
    const float sa = (q & 1) ? cp : sp;
    const float ca = (q & 1) ? sp : cp;
    *s_out = (q & 2) ? -sa : sa;
    *c_out = ((q + 1) & 2) ? -ca : ca;
}

// The routine's stores: write-through (store_result) for the one-row launch that ends with them, plain otherwise.
template <bool WRITE_THROUGH>
__device__ __forceinline__ void rope_store(uint16_t* p, uint16_t v) {
    if constexpr (WRITE_THROUGH) store_result(p, v);
    else *p = v;
}

// Called by the 64 lanes of one wave; lane i brings elements i and i + 64 of head `head`
// (0 .. n_q + 2 n_kv - 1, query heads first, then key heads, then value heads) as bf16 bits.
//   out[i]      = x[i] * cos(pos f_i) - x[i+64] * sin(pos f_i)
//   out[i + 64] = x[i+64] * cos(pos f_i) + x[i] * sin(pos f_i),     f_i = theta^(-i/64)
// where x is the head after RMSNorm (rounded to bf16, as a bf16 norm layer returns it).
// `pos`, `gain_a` and `gain_b` are *t.pos and elements lane and lane + 64 of the head's gain (q_gain for a
// query head, k_gain for a key head, unused for a value head): a caller that knows early which head
// a wave will serve loads them ahead of time.
// Sine and cosine of the rotation of elements lane and lane + 64 at position `pos`: they depend on nothing a GEMV
// computes, so a kernel that ends with the rotation can have them ready long before.
__device__ __forceinline__ void rope_angle(const RopeTarget& t, int pos, int lane, float* s, float* c) {
    const float freq = exp2f(-t.log2_theta * static_cast<float>(lane) / 64.0f);
    rope_sincos(static_cast<float>(pos) * freq, s, c);
}

template <bool WRITE_THROUGH = false>
__device__ __forceinline__ void qk_norm_rope_head_at(uint16_t a_bits, uint16_t b_bits, int head, int lane,
                                                     const RopeTarget& t, int pos, uint16_t gain_a,
                                                     uint16_t gain_b, float s, float c) {
    const bool row_ok = static_cast<unsigned>(pos) < static_cast<unsigned>(t.cache_positions);
    if (head >= t.n_q + t.n_kv) {  // value head: straight into the cache
        if (row_ok) {
            uint16_t* dst = t.v_cache + (static_cast<size_t>(pos) * t.n_kv + (head - t.n_q - t.n_kv)) * kHeadDim;
            rope_store<WRITE_THROUGH>(dst + lane, a_bits);
            rope_store<WRITE_THROUGH>(dst + lane + 64, b_bits);
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
    const float oa = xa * c - xb * s;
    const float ob = xb * c + xa * s;
    // two guarded stores rather than one store through a selected pointer (see qk_norm_rope_head)
    if (is_q) {
        uint16_t* dst = t.q_out + static_cast<size_t>(head) * kHeadDim;
        rope_store<WRITE_THROUGH>(dst + lane, f32_to_bf16(oa));
        rope_store<WRITE_THROUGH>(dst + lane + 64, f32_to_bf16(ob));
    } else if (row_ok) {
        uint16_t* dst = t.k_cache + (static_cast<size_t>(pos) * t.n_kv + (head - t.n_q)) * kHeadDim;
        rope_store<WRITE_THROUGH>(dst + lane, f32_to_bf16(oa));
        rope_store<WRITE_THROUGH>(dst + lane + 64, f32_to_bf16(ob));
    }
}

// The same with the angle worked out here.
template <bool WRITE_THROUGH = false>
__device__ __forceinline__ void qk_norm_rope_head_with(uint16_t a_bits, uint16_t b_bits, int head, int lane,
                                                       const RopeTarget& t, int pos, uint16_t gain_a,
                                                       uint16_t gain_b) {
    float s, c;
    rope_angle(t, pos, lane, &s, &c);
    qk_norm_rope_head_at<WRITE_THROUGH>(a_bits, b_bits, head, lane, t, pos, gain_a, gain_b, s, c);
}

// The same with the three operands loaded here.
__device__ __forceinline__ void qk_norm_rope_head(uint16_t a_bits, uint16_t b_bits, int head, int lane,
                                                  const RopeTarget& t) {
    // both gains are read and the values selected: a select between the two pointers is compiled to a table
    // of pointers in private memory, and a kernel with private memory is slower to start its waves
    const bool is_q = head < t.n_q;  // a value head takes k_gain and ignores it
    const uint16_t qa = t.q_gain[lane], qb = t.q_gain[lane + 64];
    const uint16_t ka = t.k_gain[lane], kb = t.k_gain[lane + 64];
    qk_norm_rope_head_with(a_bits, b_bits, head, lane, t, t.pos[0], is_q ? qa : ka, is_q ? qb : kb);
}

}  // namespace kx

#endif  // KX_ROPE_H
