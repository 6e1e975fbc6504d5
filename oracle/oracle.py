"""TEST INFRASTRUCTURE: ctypes loader of the CPU oracle (oracle/libptl_oracle.so).

Only tests, the smoke check and the benchmark's cpu_baseline leg import this.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libptl_oracle.so")
_lib = None

STRUCT_FUNCS = ["orc_mm", "orc_im2row", "orc_im2col", "orc_blocktransp", "orc_transpose_matrix", "orc_transpose",
                "orc_CHW_to_HWC", "orc_HWC_to_CHW", "orc_pad_tensor"]
LAYER_FUNCS = ["orc_conv2d_fw", "orc_conv2d_wg", "orc_conv2d_ig", "orc_conv_pw_fw", "orc_conv_pw_wg",
               "orc_conv_pw_ig", "orc_conv_dw_fw", "orc_conv_dw_wg", "orc_conv_dw_ig", "orc_linear_fw",
               "orc_linear_wg", "orc_linear_ig"]


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("oracle/libptl_oracle.so is not built (run `python oracle/build.py`)")
    lib = ctypes.CDLL(LIB_PATH)
    for dt in ("fp32", "fp16"):
        for n in STRUCT_FUNCS:
            f = getattr(lib, "%s_%s" % (n, dt))
            f.argtypes = [ctypes.c_void_p]
            f.restype = None
        for n in LAYER_FUNCS:
            f = getattr(lib, "%s_%s" % (n, dt))
            f.argtypes = [ctypes.c_void_p, ctypes.c_int]
            f.restype = None
        f = getattr(lib, "orc_conv2d_im2col_route_%s" % dt)
        f.argtypes = [ctypes.c_void_p, ctypes.c_int]
        f.restype = None
        f = getattr(lib, "orc_vect_sum_%s" % dt)
        f.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int]
        f.restype = None
    for n in ("orc_mhsa_fw_fp32", "orc_mhsa_bw_fp32"):
        f = getattr(lib, n)
        f.argtypes = [ctypes.c_void_p, ctypes.c_int]
        f.restype = None
    for n in ("orc_softmax_fw_fp32", "orc_softmax_bw_fp32"):
        f = getattr(lib, n)
        f.argtypes = [ctypes.c_void_p]
        f.restype = None
    for n in ("orc_fastexp_gist", "orc_q_rsqrt"):
        f = getattr(lib, n)
        f.argtypes = [ctypes.c_float]
        f.restype = ctypes.c_float
    for dt in ("fp32", "fp16"):
        for n in ("orc_relu", "orc_residual", "orc_avgpool", "orc_cross_entropy"):
            f = getattr(lib, "%s_%s" % (n, dt))
            f.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
            f.restype = None
        f = getattr(lib, "orc_gradient_descent_%s" % dt)
        f.argtypes = [ctypes.c_void_p]
        f.restype = None
    for name in ("orc_batch_norm_fw_fp32", "orc_batch_norm_bw_fp32", "orc_batch_norm_fw_fp16", "orc_batch_norm_bw_fp16"):
        getattr(lib, name).argtypes = [ctypes.c_void_p]
        getattr(lib, name).restype = None
    lib.orc_num_threads.restype = ctypes.c_int
    lib.orc_set_num_threads.argtypes = [ctypes.c_int]
    _lib = lib
    return lib


def call(name, dtype, args_struct, *extra):
    """Call oracle function `name`_<dtype> ('fp32' or 'fp16') on a ctypes struct."""
    getattr(load(), "%s_%s" % (name, dtype))(ctypes.byref(args_struct), *extra)
