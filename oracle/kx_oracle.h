/*
 * CPU oracle for the INT4 AWQ dequantize+GEMV path and its BF16 GEMV fallback.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing in the shipped library links, loads or calls
 * this file; it exists so that the HIP kernels can be checked against an
 * independent, obviously-correct evaluation of the closed form
 *
 *        w[k,n] = (q[k,n] - z[k/G,n]) * s[k/G,n]          y[m,n] = sum_k x[m,k] * w[k,n]
 *
 * The reference tree (/root/reference) holds no implementation of this arithmetic:
 * kuiper/include/op/matmul.h:7-9 is an empty namespace and base::DataType has no
 * 16-bit float or 4-bit member (kuiper/include/base/base.h:41-46). The functions
 * below therefore follow the closed form, and follow the reference only in style:
 * single-threaded loops over raw pointers with the stream argument ignored, as in
 * kuiper/source/op/kernel/cpu/add_kernel.cpp:5-26.
 *
 * Pin status (what the test-suite checks each function against):
 *   bf16/fp16 conversions ... exhaustive over all 65536 patterns vs torch casts
 *   pack / unpack ........... known-answer words, 8x16 exhaustive positions, and an
 *                             independent numpy restatement of the layout
 *   dequant ................. exhaustive 16 x 16 x 65536 vs numpy; closed-form
 *                             invariants (q == z, antisymmetry, s == 1)
 *   awq gemv ................ numpy brute force on small shapes, exact special
 *                             cases (one-hot x, x == 0, q == z, all ones), linearity
 *   bf16 gemv ............... torch fp32/fp64 matmul
 * No golden vector of the reference covers any of these, so with respect to the
 * reference every function here is "parity unpinned"; the checks above are
 * what the mathematics fixes.
 *
 * Packed layout (one definition for the whole repository):
 *   qweight  int32 [K, N/8]      scales  fp16 [K/G, N]      qzeros  int32 [K/G, N/8]
 *   nibble i (bits 4i..4i+3) of word (r, j) holds column 8*j + ORDER[i],
 *   ORDER = {0, 2, 4, 6, 1, 3, 5, 7}.
 */
#ifndef KX_ORACLE_H
#define KX_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar conversions (round to nearest even; NaN stays NaN, quiet) ---- */
uint16_t kxo_f32_to_bf16(float f);
float kxo_bf16_to_f32(uint16_t h);
uint16_t kxo_f32_to_f16(float f);
float kxo_f16_to_f32(uint16_t h);
void kxo_f32_to_bf16_n(const float* src, uint16_t* dst, size_t n);
void kxo_bf16_to_f32_n(const uint16_t* src, float* dst, size_t n);
void kxo_f32_to_f16_n(const float* src, uint16_t* dst, size_t n);
void kxo_f16_to_f32_n(const uint16_t* src, float* dst, size_t n);

/* ---- nibble stream ---- */
/* codes: uint8 [rows, cols] with values 0..15 (cols % 8 == 0)  ->  words: int32 [rows, cols/8] */
int kxo_awq_pack(const uint8_t* codes, int64_t rows, int64_t cols, int32_t* words);
int kxo_awq_unpack(const int32_t* words, int64_t rows, int64_t cols, uint8_t* codes);

/* ---- dequantisation: w = bf16_rne(float(q - z) * float(s)), w_bf16 is [K, N] ---- */
int kxo_awq_dequant_bf16(const int32_t* qweight, const uint16_t* scales_f16, const int32_t* qzeros,
                         int64_t K, int64_t N, int64_t group, uint16_t* w_bf16);
/* one element of the same formula, for exhaustive sweeps */
uint16_t kxo_awq_dequant_one(uint32_t q, uint32_t z, uint16_t scale_f16);

/* ---- fused dequant + GEMV ---- */
/* fp64 evaluation from the unpacked codes; y_f64 is [M, N] */
int kxo_gemv_awq_f64(const uint16_t* x_bf16, const int32_t* qweight, const uint16_t* scales_f16,
                     const int32_t* qzeros, int64_t M, int64_t K, int64_t N, int64_t group,
                     double* y_f64);
/* fp32 evaluation of w = (q - z) * s with sequential fp32 accumulation over k; y is bf16 [M, N].
 * This is also the single-threaded CPU baseline that the benchmark times. */
int kxo_gemv_awq_f32(const uint16_t* x_bf16, const int32_t* qweight, const uint16_t* scales_f16,
                     const int32_t* qzeros, int64_t M, int64_t K, int64_t N, int64_t group,
                     uint16_t* y_bf16);

/* The same for the word columns [j_begin, j_end) only (columns 8*j_begin .. 8*j_end-1 of y are
 * written): lets a caller spread one GEMV over threads.  Pinned by the full-range function, of
 * which it is the body: any split returns the same bits. */
int kxo_gemv_awq_f32_range(const uint16_t* x_bf16, const int32_t* qweight, const uint16_t* scales_f16,
                           const int32_t* qzeros, int64_t M, int64_t K, int64_t N, int64_t group,
                           int64_t j_begin, int64_t j_end, uint16_t* y_bf16);

/* ---- BF16 GEMV: y[m,n] = sum_k x[m,k] * W[n,k], W bf16 row-major [N, K] ---- */
int kxo_gemv_bf16_f64(const uint16_t* x_bf16, const uint16_t* w_bf16, int64_t M, int64_t K,
                      int64_t N, double* y_f64);
int kxo_gemv_bf16_f32(const uint16_t* x_bf16, const uint16_t* w_bf16, int64_t M, int64_t K,
                      int64_t N, uint16_t* y_bf16);

#ifdef __cplusplus
}
#endif
#endif /* KX_ORACLE_H */
