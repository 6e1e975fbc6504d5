"""MI355X-native matmul training core behind PULP-TrainLib's C entry points.

The product is libptl_hip.so (HIP kernels for gfx950 + C entry points with the
reference's names and argument structs).  This package only loads it and
mirrors the argument structs for Python callers; it contains no arithmetic
and no CPU fallback: without the built library `load()` raises.
"""
import ctypes
import os

from . import structs
from .structs import *  # noqa: F401,F403

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libptl_hip.so")
INCLUDE_DIR = os.path.join(os.path.dirname(_HERE), "include")

_lib = None

# The reference's hand-unrolled matmul variants (pulp_matmul_fp32.h:72-244, pulp_matmul_fp16.h:56-135), exported by name.
MM_VARIANTS_FP32 = ["mm_u2"] + ["mm_unroll_%s" % u for u in ("1x2", "1x4", "1x8", "2x1", "4x1", "8x1", "2x2", "2x4", "4x2", "4x4")] + [
    "mm_M_u2"] + ["mm_M_unroll_%s" % u for u in ("2x1", "4x1", "8x1", "1x2", "1x4", "1x8", "2x2", "4x2", "2x4", "4x4")]
MM_VARIANTS_FP16 = ["mm_fp16_SIMD_2x4", "mm_fp16_SIMD_4x8", "mm_fp16_unroll_8x1", "mm_fp16_unroll_4x1",
                    "mm_fp16_unroll_2x1", "mm_M_fp16_SIMD_2x4", "mm_M_fp16_SIMD_4x8"]
MV_VARIANTS_FP16 = ["mv_fp16_SIMD_2x1", "mv_fp16_SIMD_4x1", "mv_fp16_SIMD_8x1"]

# Reference-named `void f(void *args)` entry points exported by the library.
VOID_ENTRY_POINTS = [
    "pulp_conv2d_fp32_fw_cl", "pulp_conv2d_fp32_bw_cl", "pulp_conv2d_fp32_bw_param_grads_cl",
    "pulp_conv2d_fp32_bw_input_grads_cl", "pulp_conv2d_fp16_fw_cl", "pulp_conv2d_fp16_bw_cl",
    "pulp_conv2d_fp16_bw_param_grads_cl", "pulp_conv2d_fp16_bw_input_grads_cl",
    "pulp_conv_pw_fp32_fw_cl", "pulp_conv_pw_fp32_bw_cl", "pulp_conv_pw_fp32_bw_param_grads_cl",
    "pulp_conv_pw_fp32_bw_input_grads_cl", "pulp_conv_pw_fp16_fw_cl", "pulp_conv_pw_fp16_bw_cl",
    "pulp_conv_pw_fp16_bw_param_grads_cl", "pulp_conv_pw_fp16_bw_input_grads_cl",
    "pulp_conv_dw_fp32_fw_cl", "pulp_conv_dw_fp32_bw_cl", "pulp_conv_dw_fp32_bw_param_grads_cl",
    "pulp_conv_dw_fp32_bw_input_grads_cl", "pulp_conv_dw_fp16_fw_cl", "pulp_conv_dw_fp16_bw_cl",
    "pulp_conv_dw_fp16_bw_param_grads_cl", "pulp_conv_dw_fp16_bw_input_grads_cl",
    "pulp_linear_fp32_fw_cl", "pulp_linear_fp32_bw_cl", "pulp_linear_fp32_bw_param_grads_cl",
    "pulp_linear_fp32_bw_input_grads_cl", "pulp_linear_fp16_fw_cl", "pulp_linear_fp16_bw_cl",
    "pulp_linear_fp16_bw_param_grads_cl", "pulp_linear_fp16_bw_input_grads_cl",
    "mm", "mm_M", "mm_fp16", "mm_M_fp16", "mm_manager", "mm_manager_fp16",
    "im2col_conv2d_fw_kernel", "im2col_conv2d_param_grad_kernel", "pulp_linear_fp32_fw_cl_kernel",
    "pulp_linear_fp32_bw_param_grads_cl_kernel",
    "naive_conv2d_fw_kernel_CHW", "naive_conv2d_param_grad_kernel_CHW", "naive_conv2d_in_grad_kernel_CHW",
    "naive_conv2d_fw_kernel_CHW_fp16", "naive_conv2d_param_grad_kernel_CHW_fp16",
    "naive_conv2d_in_grad_kernel_CHW_fp16",
] + ["naive_conv2d_%s_kernel_CHW_k%dx%d_s2_p1%s" % (step, k, k, sfx) for sfx in ("", "_fp16") for k in (3, 5)
     for step in ("fw", "param_grad", "in_grad")] + [
    "mm_bias_add_transposed", "mm_bias_add_transposed_fp16",
] + MM_VARIANTS_FP32 + MM_VARIANTS_FP16 + MV_VARIANTS_FP16 + [
    "dw_kernel_forward", "dw_kernel_weight_grad", "dw_kernel_input_grad", "dw_kernel_forward_fp16",
    "dw_kernel_weight_grad_fp16", "dw_kernel_input_grad_fp16",
    "pulp_im2row_fp32", "pulp_im2col_fp32", "pulp_blocktransp_fp32", "pulp_im2row_fp16", "pulp_im2col_fp16",
    "pulp_blocktransp_fp16",
    "transpose_matrix", "transpose", "copy", "set_to_value", "vect_sum", "cast_fp16_tensor_to_fp32", "HWC_to_CHW",
    "CHW_to_HWC", "pad_tensor", "transpose_matrix_fp16", "transpose_fp16", "copy_fp16", "set_to_value_fp16",
    "vect_sum_fp16", "cast_fp32_tensor_to_fp16", "HWC_to_CHW_fp16", "CHW_to_HWC_fp16", "pad_tensor_fp16",
    "pulp_mhsa_fp32_fw_cl", "pulp_mhsa_fp32_bw_cl", "pulp_softmax_fp32_fw_cl", "pulp_softmax_fp32_bw_cl",
    "pulp_relu_fp32_fw_cl", "pulp_relu_fp32_bw_cl", "relu_core_fw_fp32", "relu_core_bw_fp32",
    "pulp_relu_fp16_fw_cl", "pulp_relu_fp16_bw_cl", "relu_core_fw_fp16", "relu_core_bw_fp16",
    "pulp_residualconn_fp32_fw", "pulp_sumnode_fp32_bw", "pulp_residualconn_fp32_bw",
    "pulp_residualconn_fp16_fw", "pulp_sumnode_fp16_bw", "pulp_residualconn_fp16_bw",
    "pulp_avgpool_fp32_fw_cl", "pulp_avgpool_fp32_bw_cl", "pulp_avgpool_fp16_fw_cl", "pulp_avgpool_fp16_bw_cl",
    "pulp_CrossEntropyLoss", "pulp_CrossEntropyLoss_backward", "pulp_CrossEntropyLoss_fp16",
    "pulp_CrossEntropyLoss_backward_fp16", "pulp_gradient_descent_fp32", "pulp_gradient_descent_fp16",
    "pulp_batch_norm_fp32_fw_cl", "pulp_batch_norm_parallelized_fp32_fw_cl",
]



# `int f(const args *, int nsamples, int step)` batched launchers of the layers around the matmul core.
STEP_ENTRY_POINTS = ["ptl_%s_%s_batched" % (n, dt) for n in ("relu", "residual", "avgpool", "cross_entropy")
                     for dt in ("fp32", "fp16")]
# `int f(const args *)`
PLAIN_ENTRY_POINTS = ["ptl_gradient_descent_fp32", "ptl_gradient_descent_fp16", "ptl_batch_norm_fp32_fw",
                      "ptl_batch_norm_fp32_bw", "ptl_batch_norm_fp16_fw", "ptl_batch_norm_fp16_bw"]

# `int f(const args *, int nsamples)` batched launchers.
BATCHED_ENTRY_POINTS = ["ptl_%s_%s_%s_batched" % (layer, dt, step)
                        for layer in ("conv2d", "conv_pw", "conv_dw", "linear")
                        for dt in ("fp32", "fp16") for step in ("fw", "wg", "ig")] + [
                            "ptl_linear_fp32_bw_batched", "ptl_linear_fp16_bw_batched",
                            "ptl_conv2d_fp32_bw_batched", "ptl_conv2d_fp16_bw_batched",
                            "ptl_mhsa_fp32_fw_batched", "ptl_mhsa_fp32_bw_batched",
                            "ptl_conv_dw_fp16_wg_noalloc",
                            # (const optim_args *list, int count)
                            "ptl_gradient_descent_fp32_multi", "ptl_gradient_descent_fp16_multi"]

# `int f(const BatchNorm_args *, const ptl_norm_fusion *)`
FUSED_NORM_ENTRY_POINTS = ["ptl_batch_norm_fused_%s_%s" % (dt, step) for dt in ("fp32", "fp16") for step in ("fw", "bw")]

# `int f(const Conv2D_args_fp16 *, int nsamples, [const] ptl_conv_cache *)` and the size query
CACHED_ENTRY_POINTS = ["ptl_conv2d_fp16_%s_batched_cached" % s for s in ("fw", "wg", "bw")] + ["ptl_conv2d_fp16_cache_bytes"]

# `int f(const Conv2D_args_fp16 *reader, int nsamples, ptl_conv_cache *)` and
# `int f(const Conv2D_args_fp16 *, int nsamples, ptl_conv_cache *in, ptl_conv_cache *out)`
CHAINED_ENTRY_POINTS = ["ptl_conv2d_fp16_cache_prepare", "ptl_conv2d_fp16_fw_batched_chained"]

# `int f(const Conv2D_args[_fp16] *, int nsamples, ptl_wg_batch *)` and `int f(ptl_wg_batch *)`
DEFERRED_ENTRY_POINTS = ["ptl_conv2d_%s_bw_batched_deferred" % dt for dt in ("fp16", "fp32")] + \
                        ["ptl_conv2d_%s_wg_flush" % dt for dt in ("fp16", "fp32")]

# `int f(const Conv2D_args[_fp16] *, int nsamples, ptl_norm_stats *)` and
# `int f(const BatchNorm_args *, const ptl_norm_fusion *, const ptl_norm_stats *)`
STATS_ENTRY_POINTS = ["ptl_conv2d_%s_fw_batched_stats" % dt for dt in ("fp16", "fp32")] + \
                     ["ptl_batch_norm_fused_%s_fw_stats" % dt for dt in ("fp16", "fp32")]

# `int f(const Conv2D_args[_fp16] *, int nsamples, ptl_wg_batch *, const ptl_grad_post *, ptl_norm_stats *)` and
# `int f(const BatchNorm_args *, const ptl_norm_fusion *, const ptl_norm_stats *fw, const ptl_norm_stats *bw)`
GRAD_STATS_ENTRY_POINTS = ["ptl_conv2d_%s_bw_batched_deferred_post" % dt for dt in ("fp16", "fp32")] + \
                          ["ptl_batch_norm_fused_%s_bw_stats" % dt for dt in ("fp16", "fp32")]

# `int f(const Conv2D_args[_fp16] *, int nsamples, ptl_norm_stats *, const BatchNorm_args *, const ptl_norm_fusion *,
#         const ptl_norm_stats *)`
NORMED_ENTRY_POINTS = ["ptl_conv2d_%s_fw_batched_normed" % dt for dt in ("fp16", "fp32")]

# `int f(const pool_args *, const Linear_args *, const loss_args *, int nsamples, ptl_wg_batch *)`
HEAD_ENTRY_POINTS = ["ptl_pool_linear_loss_%s_batched" % dt for dt in ("fp16", "fp32")]

OTHER_ENTRY_POINTS = ["ptl_init", "ptl_last_error", "ptl_last_status", "ptl_set_stream", "ptl_sync", "ptl_set_gemm_path",
                      "ptl_last_conv_direct", "ptl_last_gemm_streamed", "ptl_last_conv_resident", "ptl_last_gemm_tile", "ptl_timer_begin", "ptl_timer_end_ms", "ptl_mm_fp32", "ptl_mm_fp16", "ptl_copy_bytes",
                      "ptl_reserve", "ptl_reserved", "ptl_probe_mfma_fp16"]


def load():
    """Load libptl_hip.so and declare the signatures.  Raises if the library has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("libptl_hip.so is not built (run `python pulp-trainlib_amd/build.py`); "
                           "there is no fallback implementation")
    lib = ctypes.CDLL(LIB_PATH)
    for name in VOID_ENTRY_POINTS:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p]
        f.restype = None
    for name in BATCHED_ENTRY_POINTS:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_int]
        f.restype = ctypes.c_int
    for name in STEP_ENTRY_POINTS:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        f.restype = ctypes.c_int
    for name in PLAIN_ENTRY_POINTS:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p]
        f.restype = ctypes.c_int
    for name in FUSED_NORM_ENTRY_POINTS:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        f.restype = ctypes.c_int
    for name in CACHED_ENTRY_POINTS[:3]:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
        f.restype = ctypes.c_int
    lib.ptl_conv2d_fp16_cache_prepare.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    lib.ptl_conv2d_fp16_cache_prepare.restype = ctypes.c_int
    lib.ptl_conv2d_fp16_fw_batched_chained.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.ptl_conv2d_fp16_fw_batched_chained.restype = ctypes.c_int
    for name in DEFERRED_ENTRY_POINTS[:2]:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
        f.restype = ctypes.c_int
    for name in DEFERRED_ENTRY_POINTS[2:]:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p]
        f.restype = ctypes.c_int
    for name in STATS_ENTRY_POINTS[:2]:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
        f.restype = ctypes.c_int
    for name in STATS_ENTRY_POINTS[2:]:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        f.restype = ctypes.c_int
    for name in GRAD_STATS_ENTRY_POINTS[:2]:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        f.restype = ctypes.c_int
    for name in GRAD_STATS_ENTRY_POINTS[2:]:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        f.restype = ctypes.c_int
    for name in NORMED_ENTRY_POINTS:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        f.restype = ctypes.c_int
    for name in HEAD_ENTRY_POINTS:
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
        f.restype = ctypes.c_int
    lib.ptl_conv2d_fp16_cache_bytes.argtypes = [ctypes.c_void_p, ctypes.c_int]
    lib.ptl_conv2d_fp16_cache_bytes.restype = ctypes.c_size_t
    lib.ptl_init.argtypes = [ctypes.c_int]
    lib.ptl_init.restype = ctypes.c_int
    lib.ptl_last_error.argtypes = []
    lib.ptl_last_error.restype = ctypes.c_char_p
    lib.ptl_last_status.argtypes = []
    lib.ptl_last_status.restype = ctypes.c_int
    lib.ptl_set_stream.argtypes = [ctypes.c_void_p]
    lib.ptl_set_stream.restype = None
    lib.ptl_set_gemm_path.argtypes = [ctypes.c_int]
    lib.ptl_set_gemm_path.restype = None
    lib.ptl_last_conv_direct.argtypes = []
    lib.ptl_last_conv_direct.restype = ctypes.c_int
    lib.ptl_last_gemm_streamed.argtypes = []
    lib.ptl_last_gemm_streamed.restype = ctypes.c_int
    lib.ptl_last_conv_resident.argtypes = []
    lib.ptl_last_conv_resident.restype = ctypes.c_int
    lib.ptl_last_gemm_tile.argtypes = []
    lib.ptl_last_gemm_tile.restype = ctypes.c_int
    lib.ptl_sync.argtypes = []
    lib.ptl_sync.restype = ctypes.c_int
    lib.ptl_timer_begin.argtypes = []
    lib.ptl_timer_begin.restype = ctypes.c_int
    lib.ptl_timer_end_ms.argtypes = []
    lib.ptl_timer_end_ms.restype = ctypes.c_float
    for name in ("ptl_mm_fp32", "ptl_mm_fp16"):
        f = getattr(lib, name)
        f.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 4
        f.restype = ctypes.c_int
    lib.ptl_copy_bytes.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_long]
    lib.ptl_copy_bytes.restype = ctypes.c_int
    lib.ptl_reserve.argtypes = [ctypes.c_size_t, ctypes.c_size_t]
    lib.ptl_reserve.restype = ctypes.c_int
    lib.ptl_reserved.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
    lib.ptl_reserved.restype = None
    lib.ptl_probe_mfma_fp16.argtypes = [ctypes.c_int] * 4 + [ctypes.POINTER(ctypes.c_float)]
    lib.ptl_probe_mfma_fp16.restype = ctypes.c_int
    _lib = lib
    return lib


def call(name, args_struct, nsamples=None):
    """Call an entry point on a ctypes argument struct and raise on failure.

    `nsamples=None` calls the reference-named `void f(void*)` entry point `name`
    and checks ptl_last_status(); otherwise `name` is a batched launcher.
    """
    lib = load()
    if nsamples is None:
        getattr(lib, name)(ctypes.byref(args_struct))
        rc = lib.ptl_last_status()
    else:
        rc = getattr(lib, name)(ctypes.byref(args_struct), int(nsamples))
    if rc != 0:
        raise RuntimeError("%s failed (status %d): %s" % (name, rc, lib.ptl_last_error().decode()))
