/*
 * Entry points of libkx_hip.so that are not part of the drop-in boundary (include/kx_hip.h): what the
 * tests and the benchmark need to put one particular kernel under a shape.  No state is kept: the
 * choice travels with the call.
 */
#ifndef KX_INTERNAL_H
#define KX_INTERNAL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KX_POLICY_BY_SHAPE 0   /* what kx_gemv_awq_bf16 does: one row on the vector kernel with the fixed-point exchange
                                  wherever that applies, several rows on the MFMA kernel */
#define KX_POLICY_VECTOR 1     /* the vector-ALU kernel with the ordered fp32 exchange (any accepted shape): the sums of
                                  the launches with a prologue or an epilogue, bit for bit */
#define KX_POLICY_MFMA 2       /* the one-shot MFMA kernel where group size and N allow, else the vector kernel */

/* kx_gemv_awq_bf16 with the kernel chosen by the caller. */
int kx_gemv_awq_bf16_policy(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                            const int32_t* qzeros, uint16_t* y, int32_t M, int32_t K, int32_t N,
                            int32_t group_size, void* workspace, size_t workspace_bytes, void* stream,
                            int32_t policy);

#ifdef __cplusplus
}
#endif
#endif /* KX_INTERNAL_H */
