// What the GEMV kernels can do to the activations on the way in (PRO) and to the finished sums on the way
// out (EPI), and the operands those steps take.  Shared by the vector kernel (one activation row, every
// combination) and the matrix-core kernel (up to sixteen rows; SwiGLU and pre-reduced norm in, plain store
// and residual add out).
#ifndef KX_GEMV_FUSED_H
#define KX_GEMV_FUSED_H

#include "kx_common.h"

namespace kx {

// Activations may be produced on the way in instead of being read as a finished bf16 row
// (PRO below); the producing arithmetic and its rounding points are those of the stand-alone
// kernels, so a fused launch returns what the separate launches would.
constexpr int kProNone = 0;     // x is a bf16 [M, K] tensor
constexpr int kProSwiGLU = 1;   // x[m,k] = bf16( bf16(silu(a[m,k])) * b[m,k] )
constexpr int kProAddNorm = 2;  // r = bf16(a + b) (b optional), x = gain * bf16(r * rsqrt(mean(r^2) + eps))
constexpr int kProAddNormLong = 3;  // the same for rows of more than eight elements per thread
constexpr int kProAttnMerge = 4;  // x = the attention output, merged here from the per-chunk results (M = 1)
constexpr int kProPreNorm = 5;    // x = gain * bf16(a * rsqrt(mean(a^2) + eps)), the sum of squares given per 256 columns
constexpr int kNormChunks = 2;  // most 16-byte pieces of a row a thread holds for the sum of squares
constexpr int kMergeHold = 20;  // per-chunk values a thread holds per element it merges: 80 chunks in four parts
constexpr int kMergeStatsPerLane = 2;  // chunks per lane of the wave that prepares a head's factors (>= 80 / 64)

struct FusedInput {
    const uint16_t* a;     // gate, or the residual stream
    const uint16_t* b;     // up, or the delta to add to the residual stream (may be null)
    const uint16_t* gain;  // norm gain [K]
    uint16_t* r_out;       // where the updated residual stream goes (may be null); must not alias a
    int ld;                // elements between consecutive activation rows of a and b
    float eps;
    // kProAttnMerge: results of the first attention stage (layout in kx_attn_merge.h)
    const float* part_out;
    const float* part_ml;
    int nchunks;
    int heads_per_kv;
    // kProPreNorm: sums of squares of the rows of `a`, [M, sumsq_parts, 4]: per tile of 256 columns (at most
    // 64 tiles) the sums of its four quarters of 64 columns, 16-byte aligned
    const float* sumsq;
    int sumsq_parts;
};

// kEpiResidual: the finished rows o are added to the residual stream, out = bf16(in + bf16(o)), and the
// sums of squares of each new row are left per quarter of a column tile for the RMSNorm that follows:
//   sumsq[m, t, i] = Q_i = wave_sum over the 64 columns of quarter i of tile t
// (kProPreNorm forms ((Q0 + Q1) + Q2) + Q3 per tile and adds the tiles of a row with one more wave_sum,
// lane = tile).  A quarter is what one wave finishes, so no wave has to wait for another.
struct ResidualTarget {
    const uint16_t* in;   // bf16 [M, N]
    uint16_t* out;        // bf16 [M, N], may be `in`: an element is read and written by the same thread
    float* sumsq;         // [M, ceil(N / 256), 4]
};

// What happens to the finished sums (EPI below).
constexpr int kEpiStore = 0;   // y[m, n] = bf16(sum)
constexpr int kEpiQkRope = 1;  // the row is q | k | v heads of 128: per-head norm, rotation, cache append (M = 1)
constexpr int kEpiResidual = 2;  // residual add + per-tile sums of squares, see ResidualTarget
constexpr int kEpiStoreFixed = 3;  // y[n] = bf16(sum), M = 1, the K tiles meeting in 64-bit fixed point (kx_splitk_exchange.h)

}  // namespace kx

#endif  // KX_GEMV_FUSED_H
