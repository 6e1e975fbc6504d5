"""Full-size checks on the GPU through properties that do not need the (slow) oracle at BASELINE sizes:
the three steps of a layer are mutually adjoint, the batched launcher equals per-sample calls, and the batched
weight gradient is additive over a split of the batch."""
import numpy as np
import pytest
import torch

import helpers as hp

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def sync(lib):
    assert lib.ptl_sync() == 0, lib.ptl_last_error().decode()


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return ((torch.rand(shape, device=DEV, generator=g) * 2 - 1) * scale).to(dtype)


def dot(a, b):
    return float((a.double() * b.double()).sum())


def close(a, b, tol):
    return abs(a - b) <= tol * max(abs(a), abs(b), 1e-30)


@pytest.mark.parametrize("dt,tdt,tol", [("fp32", torch.float32, 1e-4), ("fp16", torch.float16, 5e-3)])
def test_conv2d_config1_batched_adjoint_and_per_sample(pkg, gpu, dt, tdt, tol):
    """BASELINE config 1 (16->32, 32x32, 3x3, pad 1) at batch 128."""
    ns, Ci, Co, H, K = 128, 16, 32, 32, 3
    x, w, g = rnd((ns, Ci, H, H), tdt, 1), rnd((Co, Ci, K, K), tdt, 2, 0.2), rnd((ns, Co, H, H), tdt, 3)
    y, dx, dw = torch.zeros_like(g), torch.zeros_like(x), torch.zeros_like(w)
    a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, g, Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1))
    for s in ("fw", "wg", "ig"):
        pkg.call("ptl_conv2d_%s_%s_batched" % (dt, s), a, ns)
    sync(gpu)
    lhs = dot(y, g)
    assert close(lhs, dot(x, dx), tol) and close(lhs, dot(w, dw), tol)
    # sample 77 through the reference-named single-sample entry points
    n = 77
    y1, dx1 = torch.zeros_like(g[n]), torch.zeros_like(x[n])
    a1, keep1 = hp.conv2d_args(pkg, x[n], dx1, w, None, y1, g[n], Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1))
    pkg.call("pulp_conv2d_%s_fw_cl" % dt, a1)
    pkg.call("pulp_conv2d_%s_bw_input_grads_cl" % dt, a1)
    sync(gpu)
    # (a single sample may be split along k differently, so equality holds up to summation order)
    lim = 1e-6 if dt == "fp32" else 2e-3
    assert float((y1.double() - y[n].double()).norm() / y[n].double().norm()) <= lim
    assert float((dx1.double() - dx[n].double()).norm() / dx[n].double().norm()) <= lim
    # weight gradient is additive over a split of the batch
    dwa, dwb = torch.zeros_like(w), torch.zeros_like(w)
    h = 48
    aa, ka = hp.conv2d_args(pkg, x[:h], None, w, dwa, None, g[:h], Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1))
    ab, kb = hp.conv2d_args(pkg, x[h:], None, w, dwb, None, g[h:], Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1))
    pkg.call("ptl_conv2d_%s_wg_batched" % dt, aa, h)
    pkg.call("ptl_conv2d_%s_wg_batched" % dt, ab, ns - h)
    sync(gpu)
    err = float((dwa.double() + dwb.double() - dw.double()).norm() / dw.double().norm())
    assert err <= (1e-5 if dt == "fp32" else 2e-3)


@pytest.mark.parametrize("dt,tdt,tol", [("fp32", torch.float32, 1e-4), ("fp16", torch.float16, 5e-3)])
def test_linear_config2_batched(pkg, gpu, dt, tdt, tol):
    """BASELINE config 2: 1024 -> 1024, batch 512."""
    ns, n = 512, 1024
    x, w, g = rnd((ns, n), tdt, 4, 0.05), rnd((n, n), tdt, 5, 0.05), rnd((ns, n), tdt, 6)
    y, dx, dw = torch.zeros_like(g), torch.zeros_like(x), torch.zeros_like(w)
    a, keep = hp.linear_args(pkg, x, dx, w, dw, y, g, n, n)
    for s in ("fw", "wg", "ig"):
        pkg.call("ptl_linear_%s_%s_batched" % (dt, s), a, ns)
    sync(gpu)
    lhs = dot(y, g)
    assert close(lhs, dot(x, dx), tol) and close(lhs, dot(w, dw), tol)
    # linearity of the forward step in the input (exact for a power-of-two factor)
    y2 = torch.zeros_like(g)
    x2 = (x * 2).contiguous()
    a2, keep2 = hp.linear_args(pkg, x2, None, w, None, y2, None, n, n)
    pkg.call("ptl_linear_%s_fw_batched" % dt, a2, ns)
    sync(gpu)
    # exact except where a result is a subnormal half (doubling then rounds differently by at most one 2^-24 step)
    assert float((y2.double() - 2 * y.double()).abs().max()) <= (0.0 if dt == "fp32" else 2.0 ** -24)
    # a single sample through the batch-1 kernels equals its row of the batched result within rounding
    n0 = 311
    y1 = torch.zeros(n, dtype=tdt, device=DEV)
    a1, keep1 = hp.linear_args(pkg, x[n0], None, w, None, y1, None, n, n)
    pkg.call("pulp_linear_%s_fw_cl" % dt, a1)
    sync(gpu)
    err = float((y1.double() - y[n0].double()).norm() / y[n0].double().norm())
    assert err <= (1e-5 if dt == "fp32" else 2e-3)


def test_depthwise_pointwise_config3_batched(pkg, gpu):
    """BASELINE config 3: depthwise 3x3 on 64x56x56 (stored pre-padded to 58x58), pointwise 64 -> 128, fp16, batch 64."""
    ns, C, Co, Hp, Ho, K = 64, 64, 128, 58, 56, 3
    tdt = torch.float16
    x, w, g = rnd((ns, C, Hp, Hp), tdt, 7), rnd((C, K, K), tdt, 8, 0.3), rnd((ns, C, Ho, Ho), tdt, 9)
    y, dx, dw = torch.zeros_like(g), torch.zeros_like(x), torch.zeros_like(w)
    a, keep = hp.dw_args(pkg, "fp16", x, dx, w, dw, y, g, C, Hp, Hp, K, K, Ho, Ho)
    for s in ("fw", "wg", "ig"):
        pkg.call("ptl_conv_dw_fp16_%s_batched" % s, a, ns)
    sync(gpu)
    lhs = dot(y, g)
    assert close(lhs, dot(x, dx), 5e-3) and close(lhs, dot(w, dw), 5e-3)
    # the depthwise output is bit-identical to torch's grouped convolution evaluated in fp32 and rounded once
    ref = torch.nn.functional.conv2d(x.float(), w.float()[:, None], groups=C).to(tdt)
    assert float((y.double() - ref.double()).norm() / ref.double().norm()) <= 1e-3

    px, pw_, pg = y, rnd((Co, C), tdt, 10, 0.2), rnd((ns, Co, Ho, Ho), tdt, 11)
    py, pdx, pdw = torch.zeros_like(pg), torch.zeros_like(px), torch.zeros_like(pw_)
    a, keep = hp.pw_args(pkg, px, pdx, pw_, pdw, py, pg, C, Co, Ho, Ho)
    for s in ("fw", "wg", "ig"):
        pkg.call("ptl_conv_pw_fp16_%s_batched" % s, a, ns)
    sync(gpu)
    lhs = dot(py, pg)
    assert close(lhs, dot(px, pdx), 5e-3) and close(lhs, dot(pw_, pdw), 5e-3)


def test_both_gemm_kernels_agree(pkg, gpu):
    """The pipelined and the staged GEMM kernel compute the same convolution."""
    ns, Ci, Co, H, K = 9, 5, 7, 13, 3
    x, w, g = rnd((ns, Ci, H, H), torch.float32, 12), rnd((Co, Ci, K, K), torch.float32, 13), rnd((ns, Co, H, H), torch.float32, 14)
    res = []
    try:
        for path in (0, 1):
            gpu.ptl_set_gemm_path(path)
            y, dx, dw = torch.zeros_like(g), torch.zeros_like(x), torch.zeros_like(w)
            a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, g, Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1))
            for s in ("fw", "wg", "ig"):
                pkg.call("ptl_conv2d_fp32_%s_batched" % s, a, ns)
            sync(gpu)
            res.append((y, dx, dw))
    finally:
        gpu.ptl_set_gemm_path(0)
    for u, v in zip(*res):
        assert float((u.double() - v.double()).norm() / v.double().norm()) <= 1e-5
