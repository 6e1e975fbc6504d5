"""ctypes mirrors of include/ptl_structs.h.

Tensor pointers are `c_void_p`, so one class serves the fp32 and the fp16
struct of the same name (their layouts differ only in the pointee type) and
host as well as device addresses.  Field order follows the C header, which
follows the reference (file:line given there).
"""
import ctypes as C

P = C.c_void_p
I = C.c_int


class Blob(C.Structure):
    _fields_ = [("data", P), ("diff", P), ("dim", I), ("W", I), ("H", I), ("C", I)]


BlobP = C.POINTER(Blob)


class Im2colArgs(C.Structure):
    _fields_ = [("input", BlobP), ("c", BlobP), ("output", BlobP), ("pBuffer", P), ("Lpad", I), ("Rpad", I),
                ("Upad", I), ("Dpad", I), ("mod", I), ("stride_w", I), ("stride_h", I), ("HWC", I), ("USE_DMA", I)]


class TranspArgs(C.Structure):
    _fields_ = [("in_matrix", P), ("out_matrix", P), ("N", I), ("M", I), ("dim", C.POINTER(I)),
                ("transposed_axes", C.POINTER(I)), ("n_dim", I)]


class LayoutArgs(C.Structure):
    _fields_ = [("tensor", BlobP), ("transp_buffer", P), ("transpose_data", I), ("transpose_grad", I)]


class BlocktranspArgs(C.Structure):
    _fields_ = [("weights", P), ("bt_weights", P), ("Cin", I), ("Cout", I), ("Hk", I), ("Wk", I), ("HWC", I)]


class CopyArgs(C.Structure):
    _fields_ = [("from_", P), ("to", P), ("size", I)]


class SetToValueArgs(C.Structure):
    _fields_ = [("to", P), ("value", C.c_float), ("size", I)]


class SetToValueArgsFp16(C.Structure):
    _fields_ = [("to", P), ("value", C.c_uint16), ("size", I)]


class VectSumArgs(C.Structure):
    _fields_ = [("op_1", P), ("op_2", P), ("dest", P), ("size", I)]


class CastArgs(C.Structure):
    _fields_ = [("source", P), ("destination", P), ("size", I)]


class PadArgs(C.Structure):
    _fields_ = [("source", P), ("dest", P), ("C", I), ("H", I), ("W", I), ("T_RPAD", I), ("T_LPAD", I),
                ("T_UPAD", I), ("T_DPAD", I), ("HWC_lay", I)]


class MatMulArgs(C.Structure):
    _fields_ = [("A", P), ("B", P), ("C", P), ("N", I), ("M", I), ("K", I), ("trans_B", I),
                ("H", I), ("W", I), ("pW", I), ("pH", I), ("pCin", I), ("pCout", I),
                ("stride_h", I), ("stride_w", I), ("Lpad", I), ("Rpad", I), ("Upad", I), ("Dpad", I),
                ("bias", P), ("bias_dim", I), ("USE_BIASES", I), ("bias_transposed", I), ("HWC", I)]


class KernelDWArgs(C.Structure):
    _fields_ = [("input", BlobP), ("weights", BlobP), ("output", BlobP), ("stride_h", I), ("stride_w", I),
                ("Lpad", I), ("Rpad", I), ("Upad", I), ("Dpad", I)]


class KernelDWArgsFp16(C.Structure):
    _fields_ = [("input", BlobP), ("weights", BlobP), ("output", BlobP)]


class MMManagerArgs(C.Structure):
    _fields_ = [("mm_args", C.POINTER(MatMulArgs)), ("mm_dw_args", P), ("layer_type", I), ("step_type", I),
                ("matmul_type", I)]


class MMBiasAddArgs(C.Structure):
    _fields_ = [("mat", P), ("bias", P), ("H", I), ("W", I), ("t", I)]


class Conv2DArgs(C.Structure):
    _fields_ = [("input", BlobP), ("coeff", BlobP), ("bias", BlobP), ("output", BlobP),
                ("Lpad", I), ("Rpad", I), ("Upad", I), ("Dpad", I), ("stride_h", I), ("stride_w", I),
                ("i2c_buffer", P), ("bt_buffer", P), ("skip_wg_grad", I), ("skip_in_grad", I), ("HWC", I),
                ("opt_matmul_type_fw", I), ("opt_matmul_type_wg", I), ("opt_matmul_type_ig", I),
                ("USE_BIASES", I), ("USE_IM2COL", I), ("USE_DMA_IM2COL", I)]


class PointWiseConvArgs(C.Structure):
    _fields_ = [("input", BlobP), ("coeff", BlobP), ("output", BlobP), ("transpose_buffer", P),
                ("skip_wg_grad", I), ("skip_in_grad", I), ("opt_matmul_type_fw", I), ("opt_matmul_type_wg", I),
                ("opt_matmul_type_ig", I), ("HWC", I)]


class DepthWiseConvArgs(C.Structure):
    _fields_ = [("input", BlobP), ("coeff", BlobP), ("output", BlobP), ("stride_h", I), ("stride_w", I),
                ("Lpad", I), ("Rpad", I), ("Upad", I), ("Dpad", I), ("skip_wg_grad", I), ("skip_in_grad", I),
                ("HWC", I)]


class DepthWiseConvArgsFp16(C.Structure):
    _fields_ = [("input", BlobP), ("coeff", BlobP), ("output", BlobP), ("Lpad", I), ("Rpad", I), ("Upad", I),
                ("Dpad", I), ("skip_wg_grad", I), ("skip_in_grad", I), ("HWC", I)]


class LinearArgs(C.Structure):
    _fields_ = [("input", BlobP), ("coeff", BlobP), ("bias", BlobP), ("output", BlobP), ("skip_wg_grad", I),
                ("skip_in_grad", I), ("opt_matmul_type_fw", I), ("opt_matmul_type_wg", I),
                ("opt_matmul_type_ig", I), ("use_biases", I)]


class SoftmaxArgs(C.Structure):
    _fields_ = [("input_data", P), ("input_diff", P), ("output_data", P), ("output_diff", P), ("H", I), ("W", I),
                ("L", I), ("n_heads", I), ("global_max", P), ("partial_exp_sum", P), ("maxes", P), ("sums", P)]


class MhsaArgs(C.Structure):
    _fields_ = [("input", BlobP), ("input_bn", BlobP), ("n_heads", I), ("opt_matmul_type_fw", I),
                ("opt_matmul_type_wg", I), ("opt_matmul_type_ig", I), ("output", BlobP), ("coeff_in_q", BlobP),
                ("coeff_in_k", BlobP), ("coeff_in_v", BlobP), ("bias_in_q", BlobP), ("bias_in_k", BlobP),
                ("bias_in_v", BlobP), ("coeff_out", BlobP), ("bias_out", BlobP), ("q", BlobP), ("k", BlobP),
                ("v", BlobP), ("attention_map", BlobP), ("temp_buffer", P), ("grad", P), ("head_buffer", BlobP),
                ("softmax_buffer", BlobP), ("global_max", P), ("partial_exp_sum", P), ("maxes", P), ("sums", P)]


class ActArgs(C.Structure):
    _fields_ = [("input", BlobP), ("output", BlobP), ("H", I), ("W", I)]


class SkipConnArgs(C.Structure):
    _fields_ = [("skip", BlobP), ("lout", BlobP), ("output", BlobP), ("skip_in_grad", I)]


class PoolArgs(C.Structure):
    _fields_ = [("input", BlobP), ("output", BlobP), ("Hker", I), ("Wker", I), ("Hstride", I), ("Wstride", I)]


class LossArgs(C.Structure):
    _fields_ = [("output", BlobP), ("target", P), ("wr_loss", P)]


class OptimArgs(C.Structure):
    _fields_ = [("weights", BlobP), ("biases", BlobP), ("learning_rate", C.c_float),
                ("weight_decay_lambda", C.c_float), ("use_biases", I)]


class OptimArgsFp16(C.Structure):
    _fields_ = [("weights", BlobP), ("biases", BlobP), ("learning_rate", C.c_uint16),
                ("weight_decay_lambda", C.c_uint16), ("use_biases", I)]


class BatchNormArgs(C.Structure):
    _fields_ = [("input", BlobP), ("output", BlobP), ("coeff", BlobP), ("bias", BlobP), ("batch_size", I),
                ("running_mean", P), ("running_var", P), ("running_stdev", P), ("freeze_running_params", I),
                ("skip_wg_grad", I), ("skip_in_grad", I), ("weight_data", P), ("bias_data", P), ("eps", P),
                ("B", I), ("C", I), ("H", I), ("W", I)]


class ConvCache(C.Structure):
    """struct ptl_conv_cache: the caller-owned copy of a layer's blocked input shared by ptl_conv2d_fp16_*_cached."""
    _fields_ = [("buf", P), ("bytes", C.c_size_t), ("valid", I), ("geometry", I * 6), ("relu", I)]


class WgBatch(C.Structure):
    """struct ptl_wg_batch: the partial sums of the small layers whose weight gradients one flush completes."""
    _fields_ = [("buf", P), ("bytes", C.c_size_t), ("used", C.c_size_t), ("count", I), ("offset", C.c_size_t * 32),
                ("grad", P * 32), ("shape", I * 256)]


class NormStats(C.Structure):
    """struct ptl_norm_stats: sums of a convolution's output per channel for the normalisation behind it."""
    _fields_ = [("part", P), ("bytes", C.c_size_t), ("count", C.c_size_t), ("parts", I), ("channels", I), ("valid", I)]


class GradPost(C.Structure):
    """struct ptl_grad_post: what ptl_conv2d_*_bw_batched_deferred_post does to its input gradient."""
    _fields_ = [("add", P), ("mask", P), ("x", P)]


class NormFusion(C.Structure):
    """struct ptl_norm_fusion_fp32 / _fp16: what ptl_batch_norm_fused_* does behind the normalisation."""
    _fields_ = [("relu", I), ("skip", P), ("skip_diff", P), ("diff2", P)]


LAYER_CONV2D, LAYER_DW_CONV, LAYER_PW_CONV, LAYER_LINEAR = 0, 1, 2, 3
STEP_FW, STEP_WGT_GRAD, STEP_IN_GRAD = 0, 1, 2


def addr(x):
    """Address of a numpy array (host) or torch tensor (host or device); None -> NULL."""
    if x is None:
        return None
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    if hasattr(x, "ctypes"):
        return x.ctypes.data
    return int(x)


def blob(data=None, diff=None, C_=1, H=1, W=1, dim=None):
    """struct blob over `data`/`diff` (numpy arrays or torch tensors, kept alive by the caller)."""
    b = Blob()
    b.data = addr(data)
    b.diff = addr(diff)
    b.C, b.H, b.W = C_, H, W
    b.dim = dim if dim is not None else C_ * H * W
    return b
