/*
 * TEST INFRASTRUCTURE - CPU oracle of the matmul-based training core.
 *
 * A plain-C restatement of the PULP-TrainLib primitives that the HIP library
 * replaces: mm, im2row/im2col, blocktranspose, direct Conv2D, pointwise,
 * depthwise, Linear, transposition/layout/padding helpers, in fp32 and in
 * IEEE fp16 with the reference's fp16 accumulation.  Only tests, the smoke
 * check and the CPU-baseline leg of the benchmark may load this library; the
 * product (libptl_hip.so) never does.
 *
 * fp16 arithmetic: the reference accumulates in its 16-bit type
 * (`fp16 temp; temp += a*b`, lib/sources/pulp_matmul_fp16.c:230-232).  Each
 * step is restated as acc = (fp16)((float)acc + (float)a * (float)b): the
 * product of two halves is exact in float, so this is a multiply-add with a
 * float-then-half rounding of the sum, i.e. the fused multiply-add a RISC-V
 * fp16 FPU performs up to double rounding.
 *
 * Pinning (see tests/test_oracle_*.py): every function is checked against
 * library routines (numpy.matmul / numpy.transpose / numpy.pad,
 * torch.nn.functional.conv2d and autograd in float64) on the closed-form
 * inputs of the reference's own tests and on seeded random inputs, against
 * brute force on tiny shapes, and through adjoint identities.  The bit-level
 * rounding sequence of the fp16 accumulation is pinned only against a numpy
 * float16 re-evaluation of the same definition: "parity unpinned" at the bit
 * level, pinned to 1e-2 against float64.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "ptl_structs.h"

/* ------------------------------- fp32 ------------------------------- */
#define T float
#define MAC(acc, a, b) ((acc) += (a) * (b))
#define NAME(x) x##_fp32
#define BLOB struct blob
#define MM_ARGS struct matMul_args
#define CONV_ARGS struct Conv2D_args
#define PW_ARGS struct PointWise_Conv_args
#define DW_ARGS struct DepthWise_Conv_args
#define LIN_ARGS struct Linear_args
#define I2C_ARGS struct im2col_args
#define BT_ARGS struct blocktransp_args
#define TR_ARGS struct transp_args
#define LAY_ARGS struct layout_args
#define PAD_ARGS struct pad_args
#define DW_SH(a) ((a)->stride_h)
#define DW_SW(a) ((a)->stride_w)
#define PW_HWC_W_CI_MAJOR 1
#include "ptl_oracle_impl.h"
#undef T
#undef MAC
#undef NAME
#undef BLOB
#undef MM_ARGS
#undef CONV_ARGS
#undef PW_ARGS
#undef DW_ARGS
#undef LIN_ARGS
#undef I2C_ARGS
#undef BT_ARGS
#undef TR_ARGS
#undef LAY_ARGS
#undef PAD_ARGS
#undef DW_SH
#undef DW_SW
#undef PW_HWC_W_CI_MAJOR

/* ------------------------------- fp16 ------------------------------- */
#define T _Float16
#define MAC(acc, a, b) ((acc) = (_Float16)((float)(acc) + (float)(a) * (float)(b)))
#define NAME(x) x##_fp16
#define BLOB struct blob_fp16
#define MM_ARGS struct matMul_args_fp16
#define CONV_ARGS struct Conv2D_args_fp16
#define PW_ARGS struct PointWise_Conv_args_fp16
#define DW_ARGS struct DepthWise_Conv_args_fp16
#define LIN_ARGS struct Linear_args_fp16
#define I2C_ARGS struct im2col_args_fp16
#define BT_ARGS struct blocktransp_args_fp16
#define TR_ARGS struct transp_args_fp16
#define LAY_ARGS struct layout_args_fp16
#define PAD_ARGS struct pad_args_fp16
#define DW_SH(a) (1)
#define DW_SW(a) (1)
#define PW_HWC_W_CI_MAJOR 0
#include "ptl_oracle_impl.h"

/* Number of OpenMP threads the loops above will use. */
#ifdef _OPENMP
#include <omp.h>
int orc_num_threads(void) { return omp_get_max_threads(); }
void orc_set_num_threads(int n) { if (n > 0) omp_set_num_threads(n); }
#else
int orc_num_threads(void) { return 1; }
void orc_set_num_threads(int n) { (void)n; }
#endif
