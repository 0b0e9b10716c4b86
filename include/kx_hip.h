/*
 * kx_hip.h - C ABI of the MI355X (gfx950) kernels behind the kuiper matmul operator.
 *
 * This is the only place where host C++ meets HIP.  Plain pointers and sizes; no C++
 * types, no torch types.  Every pointer is a DEVICE pointer unless said otherwise.
 * `stream` is a hipStream_t passed as void* (nullptr = the default stream), exactly how the
 * reference hands its stream to a kernel wrapper (kuiper/source/op/kernel/cuda/add_kernel.cu:28-48).
 *
 * Conventions shared by every entry point:
 *   - returns 0 on success, a positive hipError_t if a HIP call failed, or a negative
 *     KX_ERR_* code if the arguments were rejected before anything was launched;
 *   - never synchronises, never allocates, never frees; work is enqueued on `stream`;
 *   - 16-bit floats are passed as uint16_t bit patterns (bf16 activations / outputs,
 *     fp16 scales).
 *
 * Packed AWQ layout (group size G along K, G a multiple of 32, K a multiple of G, N of 8):
 *   qweight  int32 [K,   N/8]   nibble i (bits 4i..4i+3) of word (k, j) = code of column 8j+ORDER[i]
 *   qzeros   int32 [K/G, N/8]   same nibble order
 *   scales   fp16  [K/G, N]
 *   ORDER = {0, 2, 4, 6, 1, 3, 5, 7}
 * Dequantised weight: w[k,n] = (q[k,n] - z[k/G,n]) * s[k/G,n].
 *
 * The reference declares the operator these kernels serve but leaves it empty
 * (kuiper/include/op/matmul.h:7-9, layer slot LayerMatmul kuiper/include/op/layer.h:14); the
 * entry points below are what a kernel_interface entry in the style of
 * kuiper/source/op/kernel/kernel_interface.h:10-11 binds to.
 */
#ifndef KX_HIP_H
#define KX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KX_OK 0
#define KX_ERR_NULL_POINTER (-1)   /* a required pointer is null */
#define KX_ERR_BAD_SHAPE (-2)      /* M/K/N/group outside what the kernels accept */
#define KX_ERR_WORKSPACE (-3)      /* workspace missing or smaller than kx_gemv_*_workspace_bytes */
#define KX_ERR_ALIGNMENT (-4)      /* a pointer is not aligned as documented */
#define KX_ERR_ALIAS (-5)          /* an output overlaps an input that other workgroups still read */

#define KX_MAX_BATCH 16            /* largest M the GEMV entry points take */

/* ABI version; bumped when a signature or the layout of a struct below changes.  kx_abi_version() is what the
 * loaded library was built as: a binding compares it with the KX_ABI_VERSION it was compiled against before it
 * calls anything else (kx_chain_desc has no size field; a library of another version reads other fields). */
#define KX_ABI_VERSION 3
int kx_abi_version(void);

/* Static, human-readable text for a return code of this library (KX_ERR_* or hipError_t). */
const char* kx_error_string(int code);

/* ------------------------------------------------------------------------------------------
 * Workspace.  The fused GEMVs split K across workgroups; partial sums and per-tile arrival
 * counters live in a caller-owned device buffer so that the GEMV itself never allocates.
 *
 *   bytes = kx_gemv_workspace_bytes(M, K, N)      (same figure serves both GEMV kinds)
 *   kx_workspace_init(ws, bytes, stream)           once after allocation (zeroes the counters)
 *
 * A GEMV leaves the counters zeroed again, so one initialised workspace serves any number of
 * consecutive launches on ONE stream.  Launches that may overlap (different streams) need
 * separate workspaces.  The buffer must be 256-byte aligned.  Shapes whose partial sums would
 * take 4 GiB or more are rejected (KX_ERR_BAD_SHAPE); no Qwen3-sized projection comes near.
 * Reference counterpart: none (the reference has no split reduction); the allocator that
 * would provide the buffer is base::CUDADeviceAllocator, kuiper/source/base/alloc_cu.cpp:8-16.
 * ------------------------------------------------------------------------------------------ */
size_t kx_gemv_workspace_bytes(int32_t M, int32_t K, int32_t N);
int kx_workspace_init(void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Fused INT4 AWQ dequantise + GEMV:   y[m,n] = sum_k x[m,k] * (q[k,n] - z[k/G,n]) * s[k/G,n]
 *   x bf16 [M,K] row-major, y bf16 [M,N] row-major, fp32 accumulation, 1 <= M <= KX_MAX_BATCH.
 *   Reproducible: repeated launches are bitwise identical.  At M = 1 the partial sums of the K ranges of a
 *   column meet in 64-bit fixed point (one atomic add each: the order of arrival cannot matter), at M >= 2 as
 *   fp32 in an order fixed by (M,K,N,G).  qweight/qzeros 4-byte aligned, scales and x 16-byte aligned, y
 *   8-byte aligned.
 * Replaces: the GPU branch of the quantised matmul kernel that the reference's MatmulLayer
 * would fetch through kernel::get_matmul_kernel_awq(DeviceCUDA) (pattern:
 * kuiper/source/op/kernel/kernel_interface.cpp:6-14, call site pattern kuiper/source/op/add.cpp:47).
 * ------------------------------------------------------------------------------------------ */
int kx_gemv_awq_bf16(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                     const int32_t* qzeros, uint16_t* y, int32_t M, int32_t K, int32_t N,
                     int32_t group_size, void* workspace, size_t workspace_bytes, void* stream);

/* Two kernels implement kx_gemv_awq_bf16, chosen by shape: one on the vector ALUs and one on the matrix
 * cores (MFMA; M >= 2 when the group size is a power of two and N a multiple of sixteen).  The library keeps no state about the choice. */

/* kx_gemv_awq_bf16 for callers that cannot allocate or hand over a workspace (code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc): the split-K workspace is a static device array inside
 * the library, kx_gemv_awq_static_scratch_bytes() bytes (512 KiB of counters and slots + 8 MiB of partial sums) per GPU
 * the library runs on, held until the process ends.  Same arguments, kernels and bits as kx_gemv_awq_bf16.
 * A shape whose kx_gemv_workspace_bytes(M, K, N) exceeds the array is rejected with KX_ERR_WORKSPACE and
 * nothing is launched (every Qwen3-8B and -32B projection fits at M = 1, the seven separate 8B ones up to
 * M = 4; the fused 8B gate|up 4096 -> 24576 fits up to M = 2, the 32B-shaped fused gate|up 5120 -> 51200 at M = 1 only).
 * Calls no hipMalloc / hipFree.  The first call on a device looks the array's address up and enqueues
 * one small kernel that zeroes the counters (the array is zero when the library is loaded, so that kernel
 * restates what already holds); make that call outside stream capture all the same.  All calls on one GPU
 * share that GPU's array: calls that may overlap (different streams) race - use kx_gemv_awq_bf16 with
 * separate workspaces for those.
 * Reference counterpart: none (the reference has no split reduction and allocates through
 * base::CUDADeviceAllocator only, kuiper/source/base/alloc_cu.cpp:8-16); it exists for the callers named above. */
size_t kx_gemv_awq_static_scratch_bytes(void);
int kx_gemv_awq_bf16_static(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                            const int32_t* qzeros, uint16_t* y, int32_t M, int32_t K, int32_t N,
                            int32_t group_size, void* stream);

/* ------------------------------------------------------------------------------------------
 * The same GEMV with the activations produced on the way in, for the decode step (one launch
 * instead of two; M <= KX_MAX_BATCH).  Rounding points are those of the stand-alone kernels further
 * down; the K ranges of a column are added as fp32 in a fixed order here, so at M = 1 a call agrees with the two
 * separate calls to the rounding of that sum (kx_gemv_awq_bf16 adds them in fixed point there), at M >= 2 bit
 * for bit.
 *
 *   kx_gemv_awq_swiglu_bf16:  x[m,k] = bf16( bf16(silu(gate[m,k])) * up[m,k] ),  y = x W
 *       gate, up bf16, rows act_ld elements apart (act_ld >= K; halves of one [M, 2K] tensor or two
 *       tensors), 2-byte aligned.  The vector kernel at M = 1; at M >= 2 the matrix-core kernel, as
 *       kx_gemv_awq_bf16 chooses it (then bitwise kx_swiglu_bf16 followed by kx_gemv_awq_bf16), provided gate
 *       and up are 16-byte aligned and act_ld is a multiple of 8 (otherwise M >= 2 stays on the vector kernel,
 *       two rows per workgroup).
 *   kx_gemv_awq_addnorm_bf16 runs on the vector kernel for every M (built for M = 1).
 *   kx_gemv_awq_addnorm_bf16: r = bf16(residual + delta)   (delta may be null: r = residual)
 *                             x = gain * bf16(r * rsqrt(mean_k(r^2) + eps)),  y = x W
 *       residual, delta bf16 [M,K] (16-byte aligned), gain bf16 [K]; r is written to residual_out
 *       [M,K] when that is not null.  residual_out must differ from residual and delta
 *       (KX_ERR_ALIAS): every workgroup reads the whole incoming row.  K <= 8192.
 * These launches (and kx_gemv_awq_qkv_rope_bf16, kx_gemv_awq_attn_merge_bf16 and the chained launch with any
 * input but KX_IN_ROW) address the packed weights with 32-bit offsets: K * N / 2 < 2^31, else KX_ERR_BAD_SHAPE.
 * Replaces: LayerSwiGLU + LayerMatmul, resp. LayerAdd + LayerRMSNorm + LayerMatmul, executed back
 * to back (slots kuiper/include/op/layer.h:8-20; none of the three is implemented in the reference).
 * ------------------------------------------------------------------------------------------ */
int kx_gemv_awq_swiglu_bf16(const uint16_t* gate, const uint16_t* up, int32_t act_ld,
                            const int32_t* qweight, const uint16_t* scales, const int32_t* qzeros,
                            uint16_t* y, int32_t M, int32_t K, int32_t N, int32_t group_size,
                            void* workspace, size_t workspace_bytes, void* stream);
int kx_gemv_awq_addnorm_bf16(const uint16_t* residual, const uint16_t* delta, const uint16_t* gain,
                             float eps, uint16_t* residual_out, const int32_t* qweight,
                             const uint16_t* scales, const int32_t* qzeros, uint16_t* y, int32_t M,
                             int32_t K, int32_t N, int32_t group_size, void* workspace,
                             size_t workspace_bytes, void* stream);

/* The front of a decoder layer in one launch (M = 1): add + RMSNorm as in kx_gemv_awq_addnorm_bf16,
 * the fused q|k|v projection (N = (n_q_heads + 2 n_kv_heads) * 128, query heads first, then key
 * heads, then value heads), and on the finished row what kx_qk_norm_rope_bf16 does: per-head RMSNorm
 * of the query and key heads, rotation at *pos, queries to q_out, keys and values into row *pos of
 * the caches (which hold cache_positions rows; a position outside them writes no row).
 * Bitwise the result of kx_gemv_awq_addnorm_bf16 followed by kx_qk_norm_rope_bf16.
 * n_q_heads + 2 n_kv_heads must be even (a column tile of 256 holds whole heads); head_dim = 128.
 * Replaces: LayerAdd + LayerRMSNorm + LayerMatmul + LayerRMSNorm (heads) + LayerRope back to back
 * (slots kuiper/include/op/layer.h:8-20; not implemented in the reference). */
int kx_gemv_awq_qkv_rope_bf16(const uint16_t* residual, const uint16_t* delta, const uint16_t* gain,
                              float eps, uint16_t* residual_out, const int32_t* qweight,
                              const uint16_t* scales, const int32_t* qzeros, const uint16_t* q_gain,
                              const uint16_t* k_gain, uint16_t* q_out, uint16_t* k_cache, uint16_t* v_cache,
                              int32_t n_q_heads, int32_t n_kv_heads, int32_t head_dim, const int32_t* pos,
                              int32_t cache_positions, float rope_theta, float qk_eps, int32_t K,
                              int32_t group_size, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Chained GEMV: one launch whose activations come from the previous operator of a decoder
 * layer and whose result goes straight into the next one.  One activation row unless `rows` says otherwise.  `in_kind` selects where the activation
 * row x [K] comes from, `out_kind` what happens to the finished row o [N]; only the fields of the
 * selected kinds are read.
 *
 *   KX_IN_ROW       x                                    bf16 [K], 16-byte aligned
 *   KX_IN_SWIGLU    gate, up                             x = bf16(bf16(silu(gate)) * up)
 *   KX_IN_ATTN      attn_workspace (+ bytes), n_q_heads, n_kv_heads, max_positions
 *                                                        x = attention output merged from the workspace
 *                                                        of kx_attn_decode_partial_bf16 (K = n_q_heads * 128)
 *   KX_IN_NORM      norm_row, norm_sumsq, norm_parts, norm_gain, norm_eps
 *                                                        x = gain * bf16(row * rsqrt(sum(sumsq) / K + eps)),
 *                                                        sumsq = what KX_OUT_RESIDUAL left: float [norm_parts, 4],
 *                                                        norm_parts = ceil(K / 256), 16-byte aligned
 *   KX_OUT_ROW      y                                    y = bf16(o)
 *   KX_OUT_RESIDUAL residual_in, residual_out, sumsq_out residual_out = bf16(residual_in + bf16(o)) (may be
 *                                                        in place), sumsq_out[t, i] = sum of squares of columns
 *                                                        256 t + 64 i .. + 63 of residual_out: float
 *                                                        [ceil(N / 256), 4] (quarters past N: 0)
 *   KX_OUT_QKV_ROPE q_gain, k_gain, q_out, k_cache, v_cache, pos, rope_n_q_heads, rope_n_kv_heads,
 *                   cache_positions, rope_theta, qk_eps  as kx_gemv_awq_qkv_rope_bf16 (N = (n_q + 2 n_kv) * 128)
 *
 * The sum of squares of KX_OUT_RESIDUAL / KX_IN_NORM is added quarter by quarter and tile by tile
 * (((Q0 + Q1) + Q2) + Q3 per tile, then the tiles), an order of its own:
 * results agree with kx_add_rmsnorm_bf16 followed by the GEMV to within the rounding of that sum
 * (an occasional last-bit difference in the normalised row), not bit for bit.
 * With rows = 2 .. KX_MAX_BATCH every tensor gains a leading dimension (x [rows, K], y / residual_* [rows, N],
 * norm_sumsq [rows, norm_parts, 4], sumsq_out [rows, ceil(N / 256), 4]); gate, up and norm_row may have their rows
 * act_ld elements apart.  That form runs on the matrix-core kernel and takes KX_IN_ROW / KX_IN_SWIGLU /
 * KX_IN_NORM with any output kind (KX_OUT_QKV_ROPE: q_out [rows, n_q * 128], pos [rows], one cache pair per
 * row, see cache_stride), a power-of-two group size, N a multiple of 16, act_ld a
 * multiple of 8 and 16-byte aligned gate / up / norm_row / norm_gain; with SwiGLU input and residual output it
 * is bitwise kx_swiglu_bf16, kx_gemv_awq_bf16 and kx_add_bf16 back to back.
 * One row: always the vector kernel.  Replaces: the chain LayerMHA -> LayerMatmul -> LayerAdd -> LayerRMSNorm ->
 * LayerMatmul -> LayerSwiGLU -> LayerMatmul -> LayerAdd -> LayerRMSNorm of a decoder layer, one link
 * per call (slots kuiper/include/op/layer.h:8-20; none implemented in the reference).
 * ------------------------------------------------------------------------------------------ */
#define KX_IN_ROW 0
#define KX_IN_SWIGLU 1
#define KX_IN_ATTN 2
#define KX_IN_NORM 3
#define KX_OUT_ROW 0
#define KX_OUT_RESIDUAL 1
#define KX_OUT_QKV_ROPE 2

typedef struct kx_chain_desc {
    int32_t in_kind;
    int32_t out_kind;
    /* KX_IN_ROW */
    const uint16_t* x;
    /* KX_IN_SWIGLU */
    const uint16_t* gate;
    const uint16_t* up;
    /* KX_IN_ATTN */
    const void* attn_workspace;
    size_t attn_workspace_bytes;
    int32_t n_q_heads;
    int32_t n_kv_heads;
    int32_t max_positions;
    /* KX_IN_NORM */
    int32_t norm_parts;
    const uint16_t* norm_row;
    const float* norm_sumsq;
    const uint16_t* norm_gain;
    float norm_eps;
    /* KX_OUT_QKV_ROPE (scalars) */
    float rope_theta;
    float qk_eps;
    int32_t rope_n_q_heads;
    int32_t rope_n_kv_heads;
    int32_t cache_positions;
    /* KX_OUT_ROW */
    uint16_t* y;
    /* KX_OUT_RESIDUAL */
    const uint16_t* residual_in;
    uint16_t* residual_out;
    float* sumsq_out;
    /* KX_OUT_QKV_ROPE (pointers) */
    const uint16_t* q_gain;
    const uint16_t* k_gain;
    uint16_t* q_out;
    uint16_t* k_cache;
    uint16_t* v_cache;
    const int32_t* pos;
    /* activation rows (0 reads as 1) and, for KX_IN_SWIGLU / KX_IN_NORM, the elements between
     * consecutive rows of gate / up / norm_row (0 reads as K) */
    int32_t rows;
    int32_t act_ld;
    /* KX_OUT_QKV_ROPE with rows > 1: row m is sequence m, with position pos[m] and the cache pair that
     * starts m * cache_stride elements into k_cache / v_cache (at least cache_positions * n_kv_heads * 128) */
    size_t cache_stride;
} kx_chain_desc;

int kx_gemv_awq_chain_bf16(const kx_chain_desc* desc, const int32_t* qweight, const uint16_t* scales,
                           const int32_t* qzeros, int32_t K, int32_t N, int32_t group_size, void* workspace,
                           size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * BF16 GEMV fallback (non-quantised layers, lm_head):   y[m,n] = sum_k x[m,k] * W[n,k]
 *   W bf16 [N,K] row-major (dim0 = output features, dim1 = input features, the reading of
 *   LayerParam weights as [dim0, dim1]: kuiper/source/op/layer.cpp:256-276), K a multiple of 8,
 *   W and x 16-byte aligned, 1 <= M <= KX_MAX_BATCH.  The workspace is not used by the current
 *   kernels and may be null.
 * Replaces: the GPU branch of kernel::get_matmul_kernel(DeviceCUDA) for an unquantised
 * MatmulLayer (same dispatch pattern as above).
 * ------------------------------------------------------------------------------------------ */
int kx_gemv_bf16(const uint16_t* x, const uint16_t* w, uint16_t* y, int32_t M, int32_t K,
                 int32_t N, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Export kernels used to prove the integer side of the path bit-exactly.
 *   kx_awq_unpack_u8     words int32 [rows, cols/8] -> codes uint8 [rows, cols] (values 0..15)
 *   kx_awq_dequant_bf16  -> w bf16 [K,N], w = bf16_rne(float(q - z) * float(s)); the product is
 *                           exact in fp32, so this has exactly one rounding.
 * Reference counterpart: none; they serve the same checking role as the reference's GPU test
 * helper test/utils.cu:19-38 (a kernel that exists for tests to read results back).
 * ------------------------------------------------------------------------------------------ */
int kx_awq_unpack_u8(const int32_t* words, uint8_t* codes, int64_t rows, int64_t cols,
                     void* stream);
int kx_awq_dequant_bf16(const int32_t* qweight, const uint16_t* scales, const int32_t* qzeros,
                        uint16_t* w, int32_t K, int32_t N, int32_t group_size, void* stream);

/* ------------------------------------------------------------------------------------------
 * Supporting kernels of a Qwen3-style decode step, batch 1 (bf16 storage, fp32 arithmetic).
 * The reference reserves the layer slots (LayerRMSNorm, LayerRope, LayerMHA, LayerSwiGLU, LayerAdd,
 * LayerEmbedding: kuiper/include/op/layer.h:8-20) and leaves the operators empty
 * (kuiper/include/op/{rmsnorm,rope,mha,swiglu,embedding}.h); these are the GPU kernels a
 * get_*_kernel(DeviceCUDA) entry for them would return.  All pointers 16-byte aligned unless noted.
 *
 *   kx_rmsnorm_bf16       y[r,:] = gain * bf16(x[r,:] * rsqrt(mean(x[r,:]^2) + eps)),  n % 8 == 0
 *   kx_add_rmsnorm_bf16   x <- bf16(x + delta) in place (the residual add), then as above on the new x
 *   kx_qk_norm_rope_bf16  qkv = [q heads | k heads | v heads] x 128: RMSNorm over each q / k head with
 *                         its 128-element gain, rotary embedding at *pos (rotate-half convention,
 *                         frequencies theta^(-i/64)), q to q_out, k and v to row *pos of the caches
 *                         (bf16 [cache_positions][n_kv_heads][128]; a position outside
 *                         0 .. cache_positions-1 writes no cache row).  head_dim must be 128.
 *   kx_attn_decode_bf16   GQA attention of one query position against cache rows 0 .. *pos:
 *                         out[h,:] = softmax(q[h,:] . K[:,h/G,:] / sqrt(128)) V[:,h/G,:], G = n_q/n_kv
 *                         between 1 and 16; split over the context in chunks, merged by log-sum-exp.
 *                         `max_positions` (<= 65536) fixes the launch shape (a captured graph can be
 *                         replayed while *pos advances up to max_positions - 1) and the chunk size:
 *                         64 positions up to max_positions = 5120, 128 beyond.
 *   kx_attn_decode_partial_bf16   the first stage only: the per-chunk results stay in the workspace for
 *                         kx_gemv_awq_attn_merge_bf16 (below) to merge inside the o projection.
 *   kx_swiglu_bf16        out = bf16(silu(gate)) * up
 *   kx_add_bf16           out = a + b   (the reference's add operator, add_kernel.cu:4-12, in bf16)
 *   kx_embedding_bf16     out = table[*token, :]   (token clamped to the vocabulary)
 *   kx_argmax_bf16        *out_index = first index of the largest value (NaN ignored)
 * `pos` and `token` are DEVICE pointers to one int32, so that a captured graph sees new values.
 * ------------------------------------------------------------------------------------------ */
int kx_rmsnorm_bf16(const uint16_t* x, const uint16_t* gain, uint16_t* y, int32_t rows, int32_t n, float eps,
                    void* stream);
int kx_add_rmsnorm_bf16(uint16_t* x_inout, const uint16_t* delta, const uint16_t* gain, uint16_t* y,
                        int32_t rows, int32_t n, float eps, void* stream);
int kx_qk_norm_rope_bf16(const uint16_t* qkv, const uint16_t* q_gain, const uint16_t* k_gain, uint16_t* q_out,
                         uint16_t* k_cache, uint16_t* v_cache, int32_t n_q_heads, int32_t n_kv_heads,
                         int32_t head_dim, const int32_t* pos, int32_t cache_positions, float rope_theta, float eps,
                         void* stream);
size_t kx_attn_decode_workspace_bytes(int32_t n_q_heads, int32_t head_dim, int32_t max_positions);
int kx_attn_decode_bf16(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache, uint16_t* out,
                        int32_t n_q_heads, int32_t n_kv_heads, int32_t head_dim, const int32_t* pos,
                        int32_t max_positions, void* workspace, size_t workspace_bytes, void* stream);
int kx_attn_decode_partial_bf16(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                                int32_t n_q_heads, int32_t n_kv_heads, int32_t head_dim, const int32_t* pos,
                                int32_t max_positions, void* workspace, size_t workspace_bytes, void* stream);
/* The o projection of a decoder layer with the attention merge in its prologue (M = 1):
 * y = attn W, where attn [n_q_heads * 128] is what kx_attn_decode_bf16 would have written, merged
 * here from the workspace that kx_attn_decode_partial_bf16 filled with the same n_q_heads, n_kv_heads
 * and max_positions.  Bitwise the result of kx_attn_decode_bf16 followed by kx_gemv_awq_bf16 on the
 * vector kernel.  max_positions <= 10240 (80 chunks: a thread holds a row's per-chunk values in
 * registers); longer contexts use the two separate calls.
 * Replaces: the tail of LayerMHA + LayerMatmul back to back (kuiper/include/op/layer.h:8-20). */
int kx_gemv_awq_attn_merge_bf16(const void* attn_workspace, size_t attn_workspace_bytes, int32_t n_q_heads,
                                int32_t n_kv_heads, int32_t head_dim, int32_t max_positions,
                                const int32_t* qweight, const uint16_t* scales, const int32_t* qzeros,
                                uint16_t* y, int32_t N, int32_t group_size, void* workspace,
                                size_t workspace_bytes, void* stream);
int kx_swiglu_bf16(const uint16_t* gate, const uint16_t* up, uint16_t* out, int32_t n, void* stream);
int kx_add_bf16(const uint16_t* a, const uint16_t* b, uint16_t* out, int32_t n, void* stream);
int kx_embedding_bf16(const uint16_t* table, const int32_t* token, uint16_t* out, int32_t vocab, int32_t dim,
                      void* stream);
int kx_argmax_bf16(const uint16_t* x, int32_t n, int32_t* out_index, void* stream);

/* ------------------------------------------------------------------------------------------
 * The same for `batch` (1 .. KX_MAX_BATCH) sequences decoded together.  Row b of every activation
 * tensor belongs to sequence b; sequence b has its own position pos[b] and its own cache pair, which
 * starts b * cache_stride elements into k_cache / v_cache (cache_stride a multiple of 8 and at least
 * positions * n_kv_heads * 128).  Per sequence the arithmetic is that of the one-sequence calls, bit for bit;
 * only the attention of four or more sequences splits a cache of up to 5120 positions into chunks of 128
 * positions where the one-sequence call takes 64, and agrees with it to rounding.
 *   kx_qk_norm_rope_batch_bf16   qkv [batch, (n_q + 2 n_kv) * 128], q_out [batch, n_q * 128]
 *   kx_attn_decode_batch_bf16    q, out [batch, n_q * 128]; workspace of batch *
 *                                kx_attn_decode_workspace_bytes(...) bytes
 *   kx_embedding_rows_bf16       out[r, :] = table[tokens[r], :]
 *   kx_argmax_rows_bf16          out_index[r] = argmax of x[r * ld .. r * ld + n - 1]
 * The GEMVs of such a step take their rows through M (kx_gemv_awq_bf16, kx_gemv_bf16) or through
 * kx_chain_desc.rows.  No counterpart in the reference, whose decode slots are empty (see above).
 * ------------------------------------------------------------------------------------------ */
int kx_qk_norm_rope_batch_bf16(const uint16_t* qkv, const uint16_t* q_gain, const uint16_t* k_gain, uint16_t* q_out,
                               uint16_t* k_cache, uint16_t* v_cache, size_t cache_stride, int32_t n_q_heads,
                               int32_t n_kv_heads, int32_t head_dim, const int32_t* pos, int32_t cache_positions,
                               float rope_theta, float eps, int32_t batch, void* stream);
int kx_attn_decode_batch_bf16(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                              size_t cache_stride, uint16_t* out, int32_t n_q_heads, int32_t n_kv_heads,
                              int32_t head_dim, const int32_t* pos, int32_t max_positions, void* workspace,
                              size_t workspace_bytes, int32_t batch, void* stream);
int kx_embedding_rows_bf16(const uint16_t* table, const int32_t* tokens, uint16_t* out, int32_t vocab, int32_t dim,
                           int32_t rows, void* stream);
int kx_argmax_rows_bf16(const uint16_t* x, int32_t n, int32_t ld, int32_t* out_index, int32_t rows, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KX_HIP_H */
