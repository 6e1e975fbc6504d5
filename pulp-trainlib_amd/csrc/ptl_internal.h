/* Helpers shared between the HIP translation units and the C entry points.
 * Not part of the public ABI. */
#ifndef PTL_INTERNAL_H
#define PTL_INTERNAL_H
#include "ptl_api.h"
#ifdef __cplusplus
extern "C" {
#endif
void ptl_internal_set_status(int status);
/* mat[N x M] += bias broadcast: per_row = 0 adds bias[j] to column j,
 * per_row = 1 adds bias[i] to row i (mm_bias_add_transposed,
 * lib/sources/pulp_train_utils_fp32.c:1286). */
int ptl_internal_bias_add_fp32(float *mat, const float *bias, int N, int M, int per_row);
int ptl_internal_bias_add_fp16(fp16 *mat, const fp16 *bias, int N, int M, int per_row);
/* out[i] = sum_k mat[i*K + k] */
int ptl_internal_rowsum_fp32(const float *mat, float *out, int N, int K);
int ptl_internal_rowsum_fp16(const fp16 *mat, fp16 *out, int N, int K);
/* Row softmax with the approximate exponential (backward = 0) or its gradient (backward = 1). */
int ptl_internal_softmax_fp32(const struct softmax_args *a, int backward);
#ifdef __cplusplus
}
#endif
#endif
