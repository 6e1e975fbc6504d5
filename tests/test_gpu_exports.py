"""GPU parity of the kernel-level symbols the reference's layer entry points fork (a caller may fork them
itself): each one by name, through the C ABI, against the CPU oracle on the same seeded inputs.

fp32 within 1e-4 relative L2, fp16 within 1e-2 of the fp16-accumulating oracle; a single bias addition is one
rounded sum and is compared bit-exactly.
"""
import ctypes

import numpy as np
import pytest
import torch

import helpers as hp
from helpers import rel_l2

pytestmark = pytest.mark.gpu

TOL = {"fp32": 1e-4, "fp16": 1e-2}
DEV = "cuda:0"


def dev(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    return t.cpu().numpy()


def sync(lib):
    assert lib.ptl_sync() == 0, lib.ptl_last_error().decode()


def sfx(dt):
    return "" if dt == "fp32" else "_fp16"


def conv_mm_args(pkg, A, B, C, Ci, H, W, Co, Hk, Wk, pad, stride, bias=None):
    """matMul_args as the naive Conv2D kernels read it (lib/sources/pulp_conv2d_fp32.c:176-197): H/W the input
    size, pH/pW the filter size, pad = (L, R, U, D)."""
    m = pkg.MatMulArgs()
    m.A, m.B, m.C = pkg.addr(A), pkg.addr(B), pkg.addr(C)
    m.H, m.W, m.pH, m.pW, m.pCin, m.pCout = H, W, Hk, Wk, Ci, Co
    m.Lpad, m.Rpad, m.Upad, m.Dpad = pad
    m.stride_h, m.stride_w = stride
    if bias is not None:
        m.bias, m.USE_BIASES, m.bias_dim = pkg.addr(bias), 1, Co
    return m


def naive_case(pkg, orc, lib, dt, Ci, H, W, Co, K, pad, stride, seed, names, struct_geometry=True):
    """FW / WG / IG through the three kernel symbols `names` against the oracle's direct convolution."""
    nd = hp.np_dtype(dt)
    L, R, U, D = pad
    Ho, Wo = hp.conv_out(H, K, U, D, stride[0]), hp.conv_out(W, K, L, R, stride[1])
    x = hp.uniform(seed, (Ci, H, W), dtype=nd)
    w = hp.uniform(seed + 1, (Co, Ci, K, K), dtype=nd)
    dy = hp.uniform(seed + 2, (Co, Ho, Wo), dtype=nd)
    b = hp.uniform(seed + 3, (Co,), dtype=nd)
    y, dx, dw, db = np.zeros((Co, Ho, Wo), nd), np.zeros_like(x), np.zeros_like(w), np.zeros_like(b)
    a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, K, K, Ho, Wo, pad, stride, 0, 0, b, db)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_conv2d_" + s, dt, a, 1)
    gx, gw, gdy, gb = dev(x), dev(w), dev(dy), dev(b)
    gy, gdx, gdw, gdb = (dev(np.full(v.shape, 3, nd)) for v in (y, dx, dw, db))
    # a kernel whose name fixes the geometry must not read it from the struct: hand it nonsense there
    geo = (K, K, pad, stride) if struct_geometry else (7, 1, (5, 0, 3, 2), (3, 4))
    fw = conv_mm_args(pkg, gx, gw, gy, Ci, H, W, Co, geo[0], geo[1], geo[2], geo[3], gb)
    wg = conv_mm_args(pkg, gx, gdw, gdy, Ci, H, W, Co, geo[0], geo[1], geo[2], geo[3], gdb)
    ig = conv_mm_args(pkg, gdx, gw, gdy, Ci, H, W, Co, geo[0], geo[1], geo[2], geo[3])
    for name, m in zip(names, (fw, wg, ig)):
        pkg.call(name, m)
    sync(lib)
    for name, got, ref in (("y", gy, y), ("dw", gdw, dw), ("db", gdb, db), ("dx", gdx, dx)):
        e = rel_l2(host(got), ref)
        assert e <= TOL[dt], (name, e)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("case", [(4, 10, 10, 6, 3, (1, 1, 1, 1), (1, 1)), (3, 11, 9, 5, 3, (1, 0, 2, 1), (2, 2)),
                                  (16, 32, 32, 32, 3, (1, 1, 1, 1), (1, 1))])
def test_naive_conv2d_kernels_by_name(pkg, orc, gpu, dt, case):
    Ci, H, W, Co, K, pad, stride = case
    names = ["naive_conv2d_%s_kernel_CHW%s" % (s, sfx(dt)) for s in ("fw", "param_grad", "in_grad")]
    naive_case(pkg, orc, gpu, dt, Ci, H, W, Co, K, pad, stride, 0xC0DE0301, names)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("K", [3, 5])
@pytest.mark.parametrize("Ci,H,W,Co", [(16, 32, 32, 32), (3, 9, 13, 5), (8, 16, 16, 8)])
def test_naive_conv2d_fixed_geometry_kernels(pkg, orc, gpu, dt, K, Ci, H, W, Co):
    """_k3x3_s2_p1 / _k5x5_s2_p1: filter size, stride 2 and padding 1 come from the name
    (lib/sources/pulp_conv_naive_fp32.c:520-898), the output is ((H + 2 - K) / 2 + 1) rows."""
    names = ["naive_conv2d_%s_kernel_CHW_k%dx%d_s2_p1%s" % (s, K, K, sfx(dt)) for s in ("fw", "param_grad", "in_grad")]
    naive_case(pkg, orc, gpu, dt, Ci, H, W, Co, K, (1, 1, 1, 1), (2, 2), 0xC0DE0302, names, struct_geometry=False)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("C,H,W,K", [(8, 9, 9, 3), (64, 58, 58, 3), (16, 12, 10, 5)])
def test_dw_kernels_by_name(pkg, orc, gpu, dt, C, H, W, K):
    """dw_kernel_forward / _weight_grad / _input_grad on their kernel struct (no padding, unit stride: the
    geometry the reference's backward kernels assume, lib/sources/pulp_conv_naive_fp32.c:113-193)."""
    nd = hp.np_dtype(dt)
    Ho, Wo = H - K + 1, W - K + 1
    x, w = hp.uniform(0xC0DE0311, (C, H, W), dtype=nd), hp.uniform(0xC0DE0312, (C, K, K), dtype=nd)
    dy = hp.uniform(0xC0DE0313, (C, Ho, Wo), dtype=nd)
    y, dx, dw = np.zeros_like(dy), np.zeros_like(x), np.zeros_like(w)
    a, keep = hp.dw_args(pkg, dt, x, dx, w, dw, y, dy, C, H, W, K, K, Ho, Wo)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_conv_dw_" + s, dt, a, 1)
    gx, gw, gdy = dev(x), dev(w), dev(dy)
    gy, gdx, gdw = (dev(np.full(v.shape, 3, nd)) for v in (y, dx, dw))
    bi, bw, bo = pkg.blob(gx, gdx, C, H, W), pkg.blob(gw, gdw, 1, K, K, dim=C * K * K), pkg.blob(gy, gdy, C, Ho, Wo)
    k = pkg.KernelDWArgs() if dt == "fp32" else pkg.KernelDWArgsFp16()
    k.input, k.weights, k.output = ctypes.pointer(bi), ctypes.pointer(bw), ctypes.pointer(bo)
    if dt == "fp32":
        k.stride_h = k.stride_w = 1
    for s in ("forward", "weight_grad", "input_grad"):
        pkg.call("dw_kernel_%s%s" % (s, sfx(dt)), k)
    sync(gpu)
    for name, got, ref in (("y", gy, y), ("dw", gdw, dw), ("dx", gdx, dx)):
        e = rel_l2(host(got), ref)
        assert e <= TOL[dt], (name, e)


def bias_sum(mat, bias, per_row):
    """One rounded addition per element in the tensor's own type (float32 or float16)."""
    b = bias[:, None] if per_row else bias[None, :]
    return (mat.astype(np.float32) + b.astype(np.float32)).astype(mat.dtype)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("H,W", [(7, 5), (32, 1024), (130, 70), (1, 33)])
def test_mm_bias_add_transposed(pkg, gpu, dt, H, W):
    """mat[i][j] += bias[j] (t == 0) or bias[i] (lib/sources/pulp_train_utils_fp32.c:1286-1324): bit-exact."""
    nd = hp.np_dtype(dt)
    for t in (0, 1):
        mat = hp.uniform(0xC0DE0321, (H, W), dtype=nd)
        bias = hp.uniform(0xC0DE0322, (H if t else W,), dtype=nd)
        g = dev(mat)
        gb = dev(bias)
        a = pkg.MMBiasAddArgs()
        a.mat, a.bias, a.H, a.W, a.t = pkg.addr(g), pkg.addr(gb), H, W, t
        pkg.call("mm_bias_add_transposed" + sfx(dt), a)
        sync(gpu)
        assert np.array_equal(host(g), bias_sum(mat, bias, t))


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("N,M,K", [(32, 1024, 144), (7, 5, 3), (130, 70, 515)])
def test_mm_M_and_manager_bias_epilogue(pkg, orc, gpu, dt, N, M, K):
    """mm_M (the column-sliced twin of mm) and mm_manager with USE_BIASES == 1 in both orientations
    (lib/sources/pulp_train_utils_fp32.c:1671-1682): product, then one bias addition."""
    nd = hp.np_dtype(dt)
    A = hp.normal(0xC0DE0331, (N, K), 1.0 / np.sqrt(K), nd)
    for tb in (0, 1):
        B = hp.uniform(0xC0DE0332, (M, K) if tb else (K, M), dtype=nd)
        C = np.zeros((N, M), nd)
        orc.call("orc_mm", dt, hp.mm_args(pkg, A, B, C, N, M, K, tb))
        gA, gB, gC = dev(A), dev(B), dev(np.full((N, M), 3, nd))
        m = hp.mm_args(pkg, gA, gB, gC, N, M, K, tb)
        pkg.call("mm_M" + sfx(dt), m)
        sync(gpu)
        assert rel_l2(host(gC), C) <= TOL[dt]
        man = pkg.MMManagerArgs()
        man.mm_args = ctypes.pointer(m)
        man.layer_type, man.step_type, man.matmul_type = pkg.LAYER_LINEAR, pkg.STEP_FW, 0
        for per_row in (0, 1):
            bias = hp.uniform(0xC0DE0333, (N if per_row else M,), dtype=nd)
            gb = dev(bias)
            gC.fill_(3)
            m.bias, m.bias_dim, m.USE_BIASES, m.bias_transposed = pkg.addr(gb), bias.size, 1, per_row
            pkg.call("mm_manager" + sfx(dt), man)
            sync(gpu)
            assert rel_l2(host(gC), bias_sum(C, bias, per_row)) <= TOL[dt]
            # the epilogue is exactly one addition on top of the product the same call computed
            m.USE_BIASES = 0
            gP = dev(np.zeros((N, M), nd))
            m.C = pkg.addr(gP)
            pkg.call("mm_manager" + sfx(dt), man)
            sync(gpu)
            assert np.array_equal(host(gC), bias_sum(host(gP), bias, per_row))
            m.C = pkg.addr(gC)


def test_every_unrolled_matmul_variant_by_name(pkg, orc, gpu):
    """The hand-unrolled mm variants the reference's matmul harness forks by name (tests/test_matmul/net.c:95-186;
    lib/include/pulp_matmul_fp32.h:72-244, pulp_matmul_fp16.h:56-107): on the harness's closed-form operands
    (tests/test_matmul/utils/GM.py:81-93, 32x32x32) and on a ragged product, both orientations of B, each against the
    oracle's mm."""
    for dt, names in (("fp32", ["mm", "mm_M"] + pkg.MM_VARIANTS_FP32), ("fp16", ["mm_fp16", "mm_M_fp16"] + pkg.MM_VARIANTS_FP16)):
        nd = hp.np_dtype(dt)
        assert len(names) == (24 if dt == "fp32" else 9)
        i, j = np.meshgrid(np.arange(32), np.arange(32), indexing="ij")
        cases = [(((1.0 + (i + j + 0.1)) / 1e3).astype(nd), ((i * j + 0.1) / 64).astype(nd)),
                 (hp.uniform(0xC0DE0341, (50, 39), dtype=nd), hp.uniform(0xC0DE0342, (39, 70), dtype=nd))]
        for A, B in cases:
            (N, K), M = A.shape, B.shape[1]
            for tb in (0, 1):
                Bm = np.ascontiguousarray(B.T) if tb else B
                C = np.zeros((N, M), nd)
                orc.call("orc_mm", dt, hp.mm_args(pkg, A, Bm, C, N, M, K, tb))
                assert rel_l2(C, A.astype(np.float64) @ B.astype(np.float64)) <= TOL[dt]
                gA, gB = dev(A), dev(Bm)
                for name in names:
                    gC = dev(np.full((N, M), 3, nd))
                    pkg.call(name, hp.mm_args(pkg, gA, gB, gC, N, M, K, tb))
                    sync(gpu)
                    assert rel_l2(host(gC), C) <= TOL[dt], (name, tb)


def test_matrix_vector_variants_by_name(pkg, orc, gpu):
    """mv_fp16_SIMD_{2,4,8}x1 (lib/sources/pulp_matmul_fp16.c:1158): C[i] = sum_k A[i][k] B[k]; with M > 1 and
    trans_B set M is the vector's length; with M > 1 and trans_B clear the call is refused and C stays."""
    N, K = 37, 130
    A = hp.normal(0xC0DE0343, (N, K), 1.0 / np.sqrt(K), np.float16)
    B = hp.uniform(0xC0DE0344, (K,), dtype=np.float16)
    C = np.zeros((N, 1), np.float16)
    orc.call("orc_mm", "fp16", hp.mm_args(pkg, A, B, C, N, 1, K, 0))
    assert rel_l2(C[:, 0], A.astype(np.float64) @ B.astype(np.float64)) <= 1e-2
    gA, gB = dev(A), dev(B)
    for name in pkg.MV_VARIANTS_FP16:
        for (M, Kf, tb) in ((1, K, 0), (1, K, 1), (K, 5, 1)):  # (the last: K taken from M)
            gC = dev(np.full((N,), 3, np.float16))
            pkg.call(name, hp.mm_args(pkg, gA, gB, gC, N, M, Kf, tb))
            sync(gpu)
            assert rel_l2(host(gC), C[:, 0]) <= 1e-2, (name, M, tb)
        gC = dev(np.full((N,), 3, np.float16))
        with pytest.raises(RuntimeError):
            pkg.call(name, hp.mm_args(pkg, gA, gB, gC, N, K, 5, 0))
        sync(gpu)
        assert torch.all(gC == 3)


@pytest.mark.parametrize("hwc", [0, 1])
def test_im2col_conv2d_kernels_by_name(pkg, orc, gpu, hwc):
    """im2col_conv2d_fw_kernel = product + per-output-channel bias (rows of C in CHW, columns in HWC);
    im2col_conv2d_param_grad_kernel = product + bias gradient as the row sums of the output gradient
    (lib/sources/pulp_conv2d_fp32.c:669-812)."""
    Co, Kd, P = 32, 144, 1024
    # forward: CHW C[Co x P] = W[Co x Kd] * i2c[P x Kd]^T ; HWC C[P x Co] = i2c[P x Kd] * W[Co x Kd]^T
    Wm = hp.uniform(0xC0DE0341, (Co, Kd))
    I2c = hp.uniform(0xC0DE0342, (P, Kd))
    bias = hp.uniform(0xC0DE0343, (Co,))
    A, B = (I2c, Wm) if hwc else (Wm, I2c)
    N, M = A.shape[0], B.shape[0]
    C = np.zeros((N, M), np.float32)
    orc.call("orc_mm", "fp32", hp.mm_args(pkg, A, B, C, N, M, Kd, 1))
    gA, gB, gC, gb = dev(A), dev(B), dev(np.full((N, M), 3, np.float32)), dev(bias)
    m = hp.mm_args(pkg, gA, gB, gC, N, M, Kd, 1)
    m.bias, m.bias_dim, m.USE_BIASES, m.HWC = pkg.addr(gb), Co, 1, hwc
    man = pkg.MMManagerArgs()
    man.mm_args = ctypes.pointer(m)
    man.layer_type, man.step_type, man.matmul_type = pkg.LAYER_CONV2D, pkg.STEP_FW, 10
    pkg.call("im2col_conv2d_fw_kernel", man)
    sync(gpu)
    assert rel_l2(host(gC), bias_sum(C, bias, 0 if hwc else 1)) <= TOL["fp32"]
    if hwc:
        return
    # weight gradient: dW[Co x Kd] = dY[Co x P] * i2c[P x Kd]; db[co] = sum over pixels of dY[co]
    dY = hp.uniform(0xC0DE0344, (Co, P))
    dW = np.zeros((Co, Kd), np.float32)
    orc.call("orc_mm", "fp32", hp.mm_args(pkg, dY, I2c, dW, Co, Kd, P, 0))
    gdY, gI, gdW, gdb = dev(dY), dev(I2c), dev(np.full((Co, Kd), 3, np.float32)), dev(np.full((Co,), 3, np.float32))
    m = hp.mm_args(pkg, gdY, gI, gdW, Co, Kd, P, 0)
    m.bias, m.bias_dim, m.USE_BIASES, m.HWC = pkg.addr(gdb), Co, 1, 0
    man.mm_args = ctypes.pointer(m)
    man.step_type = pkg.STEP_WGT_GRAD
    pkg.call("im2col_conv2d_param_grad_kernel", man)
    sync(gpu)
    assert rel_l2(host(gdW), dW) <= TOL["fp32"]
    assert rel_l2(host(gdb), dY.astype(np.float64).sum(axis=1)) <= TOL["fp32"]


def test_linear_kernels_by_name(pkg, orc, gpu):
    """pulp_linear_fp32_fw_cl_kernel = mm_manager (y = W x + b through its bias epilogue);
    pulp_linear_fp32_bw_param_grads_cl_kernel = dW = dy (x) x, then the bias gradient = dy
    (lib/sources/pulp_linear_fp32.c:199-267)."""
    n_in, n_out = 1024, 96
    Wm = hp.normal(0xC0DE0351, (n_out, n_in), 1.0 / 32)
    x = hp.normal(0xC0DE0352, (n_in,), 1.0 / 32)
    b = hp.uniform(0xC0DE0353, (n_out,))
    dy = hp.uniform(0xC0DE0354, (n_out,))
    y = np.zeros((n_out,), np.float32)
    orc.call("orc_mm", "fp32", hp.mm_args(pkg, Wm, x, y, n_out, 1, n_in, 0))
    gW, gx, gb, gy = dev(Wm), dev(x), dev(b), dev(np.full((n_out,), 3, np.float32))
    m = hp.mm_args(pkg, gW, gx, gy, n_out, 1, n_in, 0)
    m.bias, m.bias_dim, m.USE_BIASES, m.bias_transposed = pkg.addr(gb), n_out, 1, 1
    man = pkg.MMManagerArgs()
    man.mm_args = ctypes.pointer(m)
    man.layer_type, man.step_type, man.matmul_type = pkg.LAYER_LINEAR, pkg.STEP_FW, 0
    pkg.call("pulp_linear_fp32_fw_cl_kernel", man)
    sync(gpu)
    assert rel_l2(host(gy), y + b) <= TOL["fp32"]
    dW = np.zeros((n_out, n_in), np.float32)
    orc.call("orc_mm", "fp32", hp.mm_args(pkg, dy, x, dW, n_out, n_in, 1, 0))
    gdy, gdW, gdb = dev(dy), dev(np.full((n_out, n_in), 3, np.float32)), dev(np.full((n_out,), 3, np.float32))
    m = hp.mm_args(pkg, gdy, gx, gdW, n_out, n_in, 1, 0)
    m.bias, m.bias_dim, m.USE_BIASES = pkg.addr(gdb), n_out, 1
    man.mm_args = ctypes.pointer(m)
    man.step_type = pkg.STEP_WGT_GRAD
    pkg.call("pulp_linear_fp32_bw_param_grads_cl_kernel", man)
    sync(gpu)
    assert rel_l2(host(gdW), dW) <= TOL["fp32"]
    assert np.array_equal(host(gdb), dy)
