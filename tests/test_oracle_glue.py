"""Pins of the oracle's ResNet-step layers against library routines (CPU only): torch relu / avg_pool2d /
cross_entropy with soft targets / batch_norm and their autograd in float64, and a numpy float64 SGD update."""
import ctypes

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import helpers as hp

TOL = {"fp32": 2e-6, "fp16": 3e-3}


def t64(a, grad=False):
    return torch.tensor(np.asarray(a, dtype=np.float64), requires_grad=grad)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
def test_relu_and_residual(pkg, orc, dt):
    lib, npd = orc.load(), hp.np_dtype(dt)
    ns, dim = 3, 77
    x = hp.uniform(0x6E01, (ns, dim)).astype(npd)
    g = hp.uniform(0x6E02, (ns, dim)).astype(npd)
    y, dx = np.zeros_like(x), np.zeros_like(x)
    a, keep = hp.act_args(pkg, x, dx, y, g, dim)
    getattr(lib, "orc_relu_" + dt)(ctypes.byref(a), ns, 0)
    getattr(lib, "orc_relu_" + dt)(ctypes.byref(a), ns, 1)
    xt = t64(x, True)
    yt = F.relu(xt)
    yt.backward(t64(g))
    assert np.array_equal(y, yt.detach().numpy().astype(npd))
    assert np.array_equal(dx, xt.grad.numpy().astype(npd))
    # residual: out = skip + lout; skip.diff += out.diff; lout.diff = out.diff
    s, l = hp.uniform(0x6E03, (ns, dim)).astype(npd), hp.uniform(0x6E04, (ns, dim)).astype(npd)
    ds0 = hp.uniform(0x6E05, (ns, dim)).astype(npd)
    ds, dl, o = ds0.copy(), np.zeros_like(s), np.zeros_like(s)
    b, keep2 = hp.skip_args(pkg, s, ds, l, dl, o, g, dim)
    for step in (0, 1, 2):
        getattr(lib, "orc_residual_" + dt)(ctypes.byref(b), ns, step)
    assert hp.rel_l2(o, s.astype(np.float64) + l) <= TOL[dt]
    assert hp.rel_l2(ds, ds0.astype(np.float64) + g) <= TOL[dt]
    assert np.array_equal(dl, g)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("geo", [(5, 8, 8, 8, 8, 8, 8), (3, 9, 7, 3, 2, 2, 1), (2, 6, 6, 2, 2, 2, 2)])
def test_avgpool(pkg, orc, dt, geo):
    lib, npd = orc.load(), hp.np_dtype(dt)
    C, H, W, Hk, Wk, Hs, Ws = geo
    ns = 2
    Ho, Wo = (H - Hk + Hs) // Hs, (W - Wk + Ws) // Ws
    x = hp.uniform(0x6E10 + H, (ns, C, H, W)).astype(npd)
    g = hp.uniform(0x6E11 + H, (ns, C, Ho, Wo)).astype(npd)
    y, dx = np.zeros((ns, C, Ho, Wo), npd), np.full((ns, C, H, W), 5, npd)
    a, keep = hp.pool_args(pkg, x, dx, y, g, C, H, W, Ho, Wo, Hk, Wk, Hs, Ws)
    getattr(lib, "orc_avgpool_" + dt)(ctypes.byref(a), ns, 0)
    getattr(lib, "orc_avgpool_" + dt)(ctypes.byref(a), ns, 1)
    xt = t64(x, True)
    yt = F.avg_pool2d(xt, (Hk, Wk), (Hs, Ws))
    yt.backward(t64(g))
    assert hp.rel_l2(y, yt.detach().numpy()) <= TOL[dt]
    assert hp.rel_l2(dx, xt.grad.numpy()) <= TOL[dt]


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
def test_cross_entropy(pkg, orc, dt):
    lib, npd = orc.load(), hp.np_dtype(dt)
    ns, ncls = 6, 10
    z = (3 * hp.normal(0x6E20, (ns, ncls))).astype(npd)
    y = np.zeros((ns, ncls), npd)
    y[np.arange(ns), np.arange(ns) % ncls] = 1
    y[5] = np.float32(0.1)  # a soft target
    loss, dz = np.zeros(ns, npd), np.zeros((ns, ncls), npd)
    a, keep = hp.loss_args(pkg, z, dz, y, loss, ncls)
    getattr(lib, "orc_cross_entropy_" + dt)(ctypes.byref(a), ns, 0)
    getattr(lib, "orc_cross_entropy_" + dt)(ctypes.byref(a), ns, 1)
    zt = t64(z, True)
    lt = F.cross_entropy(zt, t64(y), reduction="none")
    lt.sum().backward()
    assert hp.rel_l2(loss, lt.detach().numpy()) <= TOL[dt]
    assert hp.rel_l2(dz, zt.grad.numpy()) <= TOL[dt]


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("lam", [0.0, 0.05])
def test_gradient_descent(pkg, orc, dt, lam):
    lib, npd = orc.load(), hp.np_dtype(dt)
    w0, g0 = hp.uniform(0x6E30, (40, 9)).astype(npd), hp.uniform(0x6E31, (40, 9)).astype(npd)
    b0, gb0 = hp.uniform(0x6E32, (40,)).astype(npd), hp.uniform(0x6E33, (40,)).astype(npd)
    w, g, b, gb = w0.copy(), g0.copy(), b0.copy(), gb0.copy()
    lr = 0.01
    a, keep = hp.optim_args(pkg, dt, w, g, b, gb, lr, lam)
    getattr(lib, "orc_gradient_descent_" + dt)(ctypes.byref(a))
    lr_, lam_ = float(npd(lr)), float(npd(lam))
    for new, new_g, old, old_g in ((w, g, w0, g0), (b, gb, b0, gb0)):
        ge = old_g.astype(np.float64) + lam_ * old.astype(np.float64)
        assert hp.rel_l2(new_g, ge) <= TOL[dt]
        assert hp.rel_l2(new, old.astype(np.float64) - lr_ * ge) <= TOL[dt]


def test_batch_norm_forward(pkg, orc):
    lib = orc.load()
    B, C, H, W = 4, 5, 6, 7
    x = (2 * hp.normal(0x6E40, (B, C, H, W)) + 0.5).astype(np.float32)
    w, b = hp.uniform(0x6E41, (C,), 0.5, 1.5), hp.uniform(0x6E42, (C,))
    eps = np.array([1e-5], np.float32)
    y = np.zeros_like(x)
    a, keep = hp.batch_norm_args(pkg, x, y, w, b, eps, B, C, H, W)
    lib.orc_batch_norm_fw_fp32(ctypes.byref(a))
    ref = F.batch_norm(t64(x), None, None, t64(w), t64(b), training=True, eps=1e-5)
    assert hp.rel_l2(y, ref.numpy()) <= 5e-6


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
def test_batch_norm_backward_and_fp16(pkg, orc, dt):
    """The restated backward pass (and the fp16 forward) against torch batch_norm and its autograd in float64."""
    lib = orc.load()
    nd = hp.np_dtype(dt)
    B, C, H, W = 5, 6, 7, 4
    x = (1.5 * hp.normal(0x6E50, (B, C, H, W)) + 0.25).astype(nd)
    g = hp.uniform(0x6E51, (B, C, H, W)).astype(nd)
    w, b = hp.uniform(0x6E52, (C,), 0.5, 1.5).astype(nd), hp.uniform(0x6E53, (C,)).astype(nd)
    eps = np.array([1e-5], nd)
    y, dx = np.zeros_like(x), np.zeros_like(x)
    dw, db = np.zeros_like(w), np.zeros_like(b)
    a, keep = hp.batch_norm_args(pkg, x, y, w, b, eps, B, C, H, W, dx, g, dw, db)
    getattr(lib, "orc_batch_norm_fw_" + dt)(ctypes.byref(a))
    getattr(lib, "orc_batch_norm_bw_" + dt)(ctypes.byref(a))
    tx, tw, tb = t64(x).requires_grad_(), t64(w).requires_grad_(), t64(b).requires_grad_()
    ref = F.batch_norm(tx, None, None, tw, tb, training=True, eps=float(eps[0]))
    ref.backward(t64(g))
    tol = 2e-5 if dt == "fp32" else 2e-3
    assert hp.rel_l2(y, ref.detach().numpy()) <= tol
    assert hp.rel_l2(dx, tx.grad.numpy()) <= tol
    assert hp.rel_l2(dw, tw.grad.numpy()) <= tol and hp.rel_l2(db, tb.grad.numpy()) <= tol
    # the skip flags leave the corresponding outputs alone
    dx[:], dw[:], db[:] = 9, 9, 9
    a.skip_in_grad = 1
    getattr(lib, "orc_batch_norm_bw_" + dt)(ctypes.byref(a))
    assert np.all(dx == 9) and not np.any(dw == 9)
    a.skip_in_grad, a.skip_wg_grad = 0, 1
    dw[:], db[:] = 9, 9
    getattr(lib, "orc_batch_norm_bw_" + dt)(ctypes.byref(a))
    assert np.all(dw == 9) and np.all(db == 9) and not np.any(dx == 9)
