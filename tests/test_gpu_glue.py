"""GPU parity of the layers around the matmul core (ReLU, residual connection, average pooling, cross-entropy,
gradient descent, batch-norm forward) against the CPU oracle, and one residual-block training step assembled
from the library's entry points against torch autograd."""
import ctypes

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import helpers as hp

pytestmark = pytest.mark.gpu

TOL = {"fp32": 1e-4, "fp16": 1e-2}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy() if hasattr(t, "cpu") else t


@pytest.mark.parametrize("device", [True, False])
@pytest.mark.parametrize("dt", ["fp32", "fp16"])
def test_relu_residual(pkg, orc, gpu, dt, device):
    olib, npd = orc.load(), hp.np_dtype(dt)
    mk = dev if device else (lambda z: z.copy())
    ns, dim = 5, 1000
    x = hp.uniform(0x7E01, (ns, dim)).astype(npd)
    g = hp.uniform(0x7E02, (ns, dim)).astype(npd)
    ry, rdx = np.zeros_like(x), np.zeros_like(x)
    a, k = hp.act_args(pkg, x, rdx, ry, g, dim)
    for step in (0, 1):
        getattr(olib, "orc_relu_" + dt)(ctypes.byref(a), ns, step)
    y, dx = mk(np.full_like(x, 7)), mk(np.full_like(x, 7))
    b, k2 = hp.act_args(pkg, mk(x), dx, y, mk(g), dim)
    for step in (0, 1):
        assert getattr(gpu, "ptl_relu_%s_batched" % dt)(ctypes.byref(b), ns, step) == 0
    gpu.ptl_sync()
    assert np.array_equal(host(y), ry) and np.array_equal(host(dx), rdx)
    # residual connection
    s, l = hp.uniform(0x7E03, (ns, dim)).astype(npd), hp.uniform(0x7E04, (ns, dim)).astype(npd)
    ds0 = hp.uniform(0x7E05, (ns, dim)).astype(npd)
    rds, rdl, ro = ds0.copy(), np.zeros_like(s), np.zeros_like(s)
    c, k3 = hp.skip_args(pkg, s, rds, l, rdl, ro, g, dim)
    for step in (0, 1, 2):
        getattr(olib, "orc_residual_" + dt)(ctypes.byref(c), ns, step)
    ds, dl, o = mk(ds0), mk(np.full_like(s, 7)), mk(np.full_like(s, 7))
    d, k4 = hp.skip_args(pkg, mk(s), ds, mk(l), dl, o, mk(g), dim)
    for step in (0, 1, 2):
        assert getattr(gpu, "ptl_residual_%s_batched" % dt)(ctypes.byref(d), ns, step) == 0
    gpu.ptl_sync()
    assert np.array_equal(host(o), ro) and np.array_equal(host(ds), rds) and np.array_equal(host(dl), rdl)
    # skip_in_grad leaves the skip gradient alone
    d.skip_in_grad = 1
    assert getattr(gpu, "ptl_residual_%s_batched" % dt)(ctypes.byref(d), ns, 1) == 0
    gpu.ptl_sync()
    assert np.array_equal(host(ds), rds)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("geo", [(64, 8, 8, 8, 8, 8, 8), (3, 9, 7, 3, 2, 2, 1), (16, 32, 32, 2, 2, 2, 2)])
def test_avgpool(pkg, orc, gpu, dt, geo):
    olib, npd = orc.load(), hp.np_dtype(dt)
    C, H, W, Hk, Wk, Hs, Ws = geo
    ns = 3
    Ho, Wo = (H - Hk + Hs) // Hs, (W - Wk + Ws) // Ws
    x = hp.uniform(0x7E10 + H, (ns, C, H, W)).astype(npd)
    g = hp.uniform(0x7E11 + H, (ns, C, Ho, Wo)).astype(npd)
    ry, rdx = np.zeros((ns, C, Ho, Wo), npd), np.zeros((ns, C, H, W), npd)
    a, k = hp.pool_args(pkg, x, rdx, ry, g, C, H, W, Ho, Wo, Hk, Wk, Hs, Ws)
    for step in (0, 1):
        getattr(olib, "orc_avgpool_" + dt)(ctypes.byref(a), ns, step)
    y, dx = dev(np.full_like(ry, 7)), dev(np.full_like(rdx, 7))
    b, k2 = hp.pool_args(pkg, dev(x), dx, y, dev(g), C, H, W, Ho, Wo, Hk, Wk, Hs, Ws)
    for step in (0, 1):
        assert getattr(gpu, "ptl_avgpool_%s_batched" % dt)(ctypes.byref(b), ns, step) == 0
    gpu.ptl_sync()
    assert hp.rel_l2(host(y), ry) <= TOL[dt]
    assert hp.rel_l2(host(dx), rdx) <= TOL[dt]
    # a window that does not match the output size is rejected and leaves the output alone
    b.Hker = Hk + 1
    assert getattr(gpu, "ptl_avgpool_%s_batched" % dt)(ctypes.byref(b), ns, 0) == 1


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("ncls", [10, 200])
def test_cross_entropy(pkg, orc, gpu, dt, ncls):
    olib, npd = orc.load(), hp.np_dtype(dt)
    ns = 37
    z = (3 * hp.normal(0x7E20, (ns, ncls))).astype(npd)
    y = np.zeros((ns, ncls), npd)
    y[np.arange(ns), (7 * np.arange(ns)) % ncls] = 1
    y[5] = npd(1.0 / ncls)
    rl, rdz = np.zeros(ns, npd), np.zeros((ns, ncls), npd)
    a, k = hp.loss_args(pkg, z, rdz, y, rl, ncls)
    for step in (0, 1):
        getattr(olib, "orc_cross_entropy_" + dt)(ctypes.byref(a), ns, step)
    loss, dz = np.full(ns, 7, npd), np.full((ns, ncls), 7, npd)
    b, k2 = hp.loss_args(pkg, z, dz, y, loss, ncls)  # host pointers
    for step in (0, 1):
        assert getattr(gpu, "ptl_cross_entropy_%s_batched" % dt)(ctypes.byref(b), ns, step) == 0
    assert hp.rel_l2(loss, rl) <= TOL[dt]
    assert hp.rel_l2(dz, rdz) <= TOL[dt]


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("lam", [0.0, 0.05])
def test_gradient_descent(pkg, orc, gpu, dt, lam):
    olib, npd = orc.load(), hp.np_dtype(dt)
    w0, g0 = hp.uniform(0x7E30, (64, 27)).astype(npd), hp.uniform(0x7E31, (64, 27)).astype(npd)
    b0, gb0 = hp.uniform(0x7E32, (64,)).astype(npd), hp.uniform(0x7E33, (64,)).astype(npd)
    rw, rg, rb, rgb = w0.copy(), g0.copy(), b0.copy(), gb0.copy()
    a, k = hp.optim_args(pkg, dt, rw, rg, rb, rgb, 0.01, lam)
    getattr(olib, "orc_gradient_descent_" + dt)(ctypes.byref(a))
    w, g, b, gb = dev(w0), dev(g0), dev(b0), dev(gb0)
    c, k2 = hp.optim_args(pkg, dt, w, g, b, gb, 0.01, lam)
    getattr(gpu, "pulp_gradient_descent_" + dt)(ctypes.byref(c))
    assert gpu.ptl_last_status() == 0, gpu.ptl_last_error().decode()
    gpu.ptl_sync()
    for got, ref in ((w, rw), (g, rg), (b, rb), (gb, rgb)):
        assert hp.rel_l2(host(got), ref) <= (1e-6 if dt == "fp32" else 2e-3)


def test_batch_norm_forward(pkg, orc, gpu):
    B, C, H, W = 8, 16, 9, 11
    x = (2 * hp.normal(0x7E40, (B, C, H, W)) + 0.5).astype(np.float32)
    w, b = hp.uniform(0x7E41, (C,), 0.5, 1.5), hp.uniform(0x7E42, (C,))
    eps = np.array([1e-5], np.float32)
    ry = np.zeros_like(x)
    a, k = hp.batch_norm_args(pkg, x, ry, w, b, eps, B, C, H, W)
    orc.load().orc_batch_norm_fw_fp32(ctypes.byref(a))
    y = np.full_like(x, 7)
    c, k2 = hp.batch_norm_args(pkg, x, y, w, b, eps, B, C, H, W)
    gpu.pulp_batch_norm_fp32_fw_cl(ctypes.byref(c))
    assert gpu.ptl_last_status() == 0, gpu.ptl_last_error().decode()
    assert hp.rel_l2(y, ry) <= 1e-5


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("B,C,H,W", [(8, 16, 9, 11), (128, 16, 32, 32), (3, 70, 8, 8)])
def test_batch_norm_training_passes(pkg, orc, gpu, dt, B, C, H, W):
    """Forward and backward in both types against the oracle (whose backward is pinned against torch autograd)."""
    nd = hp.np_dtype(dt)
    x = (1.5 * hp.normal(0x7E60, (B, C, H, W)) + 0.25).astype(nd)
    g = hp.uniform(0x7E61, (B, C, H, W)).astype(nd)
    w, b = hp.uniform(0x7E62, (C,), 0.5, 1.5).astype(nd), hp.uniform(0x7E63, (C,)).astype(nd)
    eps = np.array([1e-5], nd)
    ry, rdx, rdw, rdb = np.zeros_like(x), np.zeros_like(x), np.zeros_like(w), np.zeros_like(b)
    a, k = hp.batch_norm_args(pkg, x, ry, w, b, eps, B, C, H, W, rdx, g, rdw, rdb)
    getattr(orc.load(), "orc_batch_norm_fw_" + dt)(ctypes.byref(a))
    getattr(orc.load(), "orc_batch_norm_bw_" + dt)(ctypes.byref(a))
    gx, gg, gw, gb, geps = dev(x), dev(g), dev(w), dev(b), dev(eps)
    y, dx = torch.full_like(gx, 7), torch.full_like(gx, 7)
    dw, db = torch.full_like(gw, 7), torch.full_like(gb, 7)
    c, k2 = hp.batch_norm_args(pkg, gx, y, gw, gb, geps, B, C, H, W, dx, gg, dw, db)
    assert getattr(gpu, "ptl_batch_norm_%s_fw" % dt)(ctypes.byref(c)) == 0, gpu.ptl_last_error().decode()
    assert getattr(gpu, "ptl_batch_norm_%s_bw" % dt)(ctypes.byref(c)) == 0, gpu.ptl_last_error().decode()
    gpu.ptl_sync()
    tol = 1e-4 if dt == "fp32" else 1e-2
    for got, ref in ((y, ry), (dx, rdx), (dw, rdw), (db, rdb)):
        assert hp.rel_l2(host(got), ref) <= tol
    dx.fill_(9), dw.fill_(9), db.fill_(9)
    c.skip_in_grad = 1
    assert getattr(gpu, "ptl_batch_norm_%s_bw" % dt)(ctypes.byref(c)) == 0
    gpu.ptl_sync()
    assert bool(torch.all(dx == 9)) and hp.rel_l2(host(dw), rdw) <= tol and hp.rel_l2(host(db), rdb) <= tol
    c.skip_in_grad, c.skip_wg_grad = 0, 1
    dw.fill_(9), db.fill_(9)
    assert getattr(gpu, "ptl_batch_norm_%s_bw" % dt)(ctypes.byref(c)) == 0
    gpu.ptl_sync()
    assert bool(torch.all(dw == 9)) and bool(torch.all(db == 9)) and hp.rel_l2(host(dx), rdx) <= tol


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("B,C,H,W", [(8, 16, 9, 11), (128, 16, 32, 32), (5, 70, 8, 8)])
@pytest.mark.parametrize("relu,skip,second,keep", [(1, 1, 1, 1), (1, 0, 0, 0), (0, 1, 0, 1), (1, 1, 0, 0), (1, 0, 1, 1)])
def test_batch_norm_fused_with_residual_and_relu(pkg, gpu, dt, B, C, H, W, relu, skip, second, keep):
    """out = [relu](bn(x) [+ skip]) and its backward from dy [+ dy2] in one call each, against torch autograd in
    float64 on the same rounded inputs (tolerances: a few roundings of the result type)."""
    import torch.nn.functional as F
    nd = hp.np_dtype(dt)
    x = (1.5 * hp.normal(0x7F60, (B, C, H, W)) + 0.25).astype(nd)
    sk = hp.normal(0x7F64, (B, C, H, W)).astype(nd)
    g1, g2 = hp.uniform(0x7F61, (B, C, H, W)).astype(nd), hp.uniform(0x7F65, (B, C, H, W)).astype(nd)
    w, b = hp.uniform(0x7F62, (C,), 0.5, 1.5).astype(nd), hp.uniform(0x7F63, (C,)).astype(nd)
    eps = np.array([1e-5], nd)
    gx, gsk, gg1, gg2, gw, gb, geps = dev(x), dev(sk), dev(g1), dev(g2), dev(w), dev(b), dev(eps)
    y, dx, ds = torch.full_like(gx, 7), torch.full_like(gx, 7), torch.full_like(gx, 7)
    dw, db = torch.full_like(gw, 7), torch.full_like(gb, 7)
    c, k2 = hp.batch_norm_args(pkg, gx, y, gw, gb, geps, B, C, H, W, dx, gg1, dw, db)
    f = pkg.NormFusion()
    f.relu = relu
    f.skip = pkg.addr(gsk) if skip else None
    f.skip_diff = pkg.addr(ds) if keep else None
    f.diff2 = pkg.addr(gg2) if second else None
    assert getattr(gpu, "ptl_batch_norm_fused_%s_fw" % dt)(ctypes.byref(c), ctypes.byref(f)) == 0, gpu.ptl_last_error().decode()
    assert getattr(gpu, "ptl_batch_norm_fused_%s_bw" % dt)(ctypes.byref(c), ctypes.byref(f)) == 0, gpu.ptl_last_error().decode()
    gpu.ptl_sync()
    # reference
    tx = torch.tensor(x.astype(np.float64), requires_grad=True)
    tw, tb = torch.tensor(w.astype(np.float64), requires_grad=True), torch.tensor(b.astype(np.float64), requires_grad=True)
    pre = F.batch_norm(tx, None, None, tw, tb, training=True, eps=float(eps[0]))
    if skip:
        pre = pre + torch.tensor(sk.astype(np.float64))
    out = torch.relu(pre) if relu else pre
    gin = g1.astype(np.float64) + (g2.astype(np.float64) if second else 0.0)
    gin = gin.astype(nd).astype(np.float64)  # the sum is a tensor of the layer's type
    out.backward(torch.tensor(gin))
    tol = 2e-5 if dt == "fp32" else 2e-3
    got_y = host(y).astype(np.float64)
    assert hp.rel_l2(got_y, out.detach().numpy()) <= tol
    # the mask the library used is its own rounded forward result; where torch's result is within rounding of 0
    # the two may differ, so the gradient reference takes the library's sign pattern
    mask = (got_y > 0) if relu else np.ones_like(got_y, bool)
    gref = np.where(mask, gin, 0.0)
    if keep:
        assert np.array_equal(host(ds).astype(np.float64), gref)
    tx2 = torch.tensor(x.astype(np.float64), requires_grad=True)
    tw2, tb2 = torch.tensor(w.astype(np.float64), requires_grad=True), torch.tensor(b.astype(np.float64), requires_grad=True)
    F.batch_norm(tx2, None, None, tw2, tb2, training=True, eps=float(eps[0])).backward(torch.tensor(gref))
    for got, ref in ((dx, tx2.grad), (dw, tw2.grad), (db, tb2.grad)):
        assert hp.rel_l2(host(got).astype(np.float64), ref.numpy()) <= tol
    if not keep:
        assert bool(torch.all(ds == 7))


def test_reference_named_single_sample_entry_points(pkg, orc, gpu):
    dim = 300
    x, g = hp.uniform(0x7E50, (dim,)), hp.uniform(0x7E51, (dim,))
    y, dx = np.zeros_like(x), np.zeros_like(x)
    a, k = hp.act_args(pkg, x, dx, y, g, dim)
    gpu.pulp_relu_fp32_fw_cl(ctypes.byref(a))
    gpu.relu_core_bw_fp32(ctypes.byref(a))
    assert gpu.ptl_last_status() == 0
    assert np.array_equal(y, np.maximum(x, 0)) and np.array_equal(dx, np.where(x > 0, g, 0))
    z = hp.normal(0x7E52, (10,))
    t = np.zeros(10, np.float32)
    t[3] = 1
    loss, dz = np.zeros(1, np.float32), np.zeros(10, np.float32)
    b, k2 = hp.loss_args(pkg, z, dz, t, loss, 10)
    gpu.pulp_CrossEntropyLoss(ctypes.byref(b))
    gpu.pulp_CrossEntropyLoss_backward(ctypes.byref(b))
    zt = torch.tensor(z.astype(np.float64), requires_grad=True)
    lt = F.cross_entropy(zt[None], torch.tensor([3]))
    lt.backward()
    assert abs(loss[0] - lt.item()) < 1e-5 and hp.rel_l2(dz, zt.grad.numpy()) < 1e-5


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
def test_residual_block_training_step(pkg, gpu, dt):
    """conv3x3 -> ReLU -> conv3x3 -> (+ input) -> ReLU -> global average pool -> linear -> cross-entropy, the
    backward pass through all of it and one SGD update, from the library's entry points, against torch autograd
    in float64 on the same (rounded) inputs."""
    npd = hp.np_dtype(dt)
    # fp16: every activation and gradient tensor of the chain is stored in half precision (the pooled gradient is
    # divided by 64 and sits near the subnormal range), so the deepest gradients carry a few percent of rounding
    tol = {"fp32": 1e-4, "fp16": 6e-2}[dt]
    ns, C, H, ncls, lr = 6, 16, 8, 10, 0.05
    x0 = hp.uniform(0x7E60, (ns, C, H, H)).astype(npd)
    w1 = (hp.uniform(0x7E61, (C, C, 3, 3)) * 0.2).astype(npd)
    w2 = (hp.uniform(0x7E62, (C, C, 3, 3)) * 0.2).astype(npd)
    wl = (hp.uniform(0x7E63, (ncls, C)) * 0.5).astype(npd)
    tgt = np.zeros((ns, ncls), npd)
    tgt[np.arange(ns), np.arange(ns) % ncls] = 1
    z = lambda *s: torch.zeros(*s, dtype=torch.float16 if dt == "fp16" else torch.float32, device="cuda")
    X0, W1, W2, WL, T = dev(x0), dev(w1), dev(w2), dev(wl), dev(tgt)
    dX0, dW1, dW2, dWL = z(ns, C, H, H), z(C, C, 3, 3), z(C, C, 3, 3), z(ncls, C)
    A1, dA1, R1, dR1 = z(ns, C, H, H), z(ns, C, H, H), z(ns, C, H, H), z(ns, C, H, H)
    A2, dA2, S, dS, R2, dR2 = (z(ns, C, H, H) for _ in range(6))
    Pl, dPl, Z, dZ, loss = z(ns, C), z(ns, C), z(ns, ncls), z(ns, ncls), z(ns)
    dim = C * H * H
    c1, k1 = hp.conv2d_args(pkg, X0, dX0, W1, dW1, A1, dA1, C, H, H, C, 3, 3, H, H, (1, 1, 1, 1))
    r1, k2 = hp.act_args(pkg, A1, dA1, R1, dR1, dim)
    c2, k3 = hp.conv2d_args(pkg, R1, dR1, W2, dW2, A2, dA2, C, H, H, C, 3, 3, H, H, (1, 1, 1, 1))
    sk, k4 = hp.skip_args(pkg, X0, dX0, A2, dA2, S, dS, dim)
    r2, k5 = hp.act_args(pkg, S, dS, R2, dR2, dim)
    pl, k6 = hp.pool_args(pkg, R2, dR2, Pl, dPl, C, H, H, 1, 1, H, H, H, H)
    ln, k7 = hp.linear_args(pkg, Pl, dPl, WL, dWL, Z, dZ, C, ncls)
    ls, k8 = hp.loss_args(pkg, Z, dZ, T, loss, ncls)
    ok = lambda rc: (rc == 0) or pytest.fail(gpu.ptl_last_error().decode())
    ref = ctypes.byref
    L = lambda name: getattr(gpu, name.replace("DT", dt))
    # forward
    ok(L("ptl_conv2d_DT_fw_batched")(ref(c1), ns))
    ok(L("ptl_relu_DT_batched")(ref(r1), ns, 0))
    ok(L("ptl_conv2d_DT_fw_batched")(ref(c2), ns))
    ok(L("ptl_residual_DT_batched")(ref(sk), ns, 0))
    ok(L("ptl_relu_DT_batched")(ref(r2), ns, 0))
    ok(L("ptl_avgpool_DT_batched")(ref(pl), ns, 0))
    ok(L("ptl_linear_DT_fw_batched")(ref(ln), ns))
    ok(L("ptl_cross_entropy_DT_batched")(ref(ls), ns, 0))
    # backward
    ok(L("ptl_cross_entropy_DT_batched")(ref(ls), ns, 1))
    ok(L("ptl_linear_DT_bw_batched")(ref(ln), ns))
    ok(L("ptl_avgpool_DT_batched")(ref(pl), ns, 1))
    ok(L("ptl_relu_DT_batched")(ref(r2), ns, 1))
    ok(L("ptl_residual_DT_batched")(ref(sk), ns, 2))  # dA2 = dS
    ok(L("ptl_conv2d_DT_wg_batched")(ref(c2), ns))
    ok(L("ptl_conv2d_DT_ig_batched")(ref(c2), ns))
    ok(L("ptl_relu_DT_batched")(ref(r1), ns, 1))
    ok(L("ptl_conv2d_DT_wg_batched")(ref(c1), ns))
    ok(L("ptl_conv2d_DT_ig_batched")(ref(c1), ns))   # dX0 = conv path
    ok(L("ptl_residual_DT_batched")(ref(sk), ns, 1))  # dX0 += dS (skip path)
    gpu.ptl_sync()
    grads = {n: host(t).astype(np.float64) for n, t in (("w1", dW1), ("w2", dW2), ("wl", dWL), ("x", dX0))}
    # update
    for Wt, dWt in ((W1, dW1), (W2, dW2), (WL, dWL)):
        o, ko = hp.optim_args(pkg, dt, Wt, dWt, None, None, lr, 0.0)
        ok(L("ptl_gradient_descent_DT")(ref(o)))
    gpu.ptl_sync()
    # torch float64
    xt = torch.tensor(x0.astype(np.float64), requires_grad=True)
    p = [torch.tensor(v.astype(np.float64), requires_grad=True) for v in (w1, w2, wl)]
    a1 = F.relu(F.conv2d(xt, p[0], padding=1))
    s = F.conv2d(a1, p[1], padding=1) + xt
    pooled = F.relu(s).mean((2, 3))
    logits = pooled @ p[2].t()
    lt = F.cross_entropy(logits, torch.tensor(tgt.astype(np.float64)), reduction="none")
    lt.sum().backward()
    assert hp.rel_l2(host(loss), lt.detach().numpy()) <= tol
    assert hp.rel_l2(host(Z), logits.detach().numpy()) <= tol
    for n, t in (("w1", p[0]), ("w2", p[1]), ("wl", p[2]), ("x", xt)):
        assert hp.rel_l2(grads[n], t.grad.numpy()) <= tol, n
    lr_ = float(npd(lr))
    for Wt, t in ((W1, p[0]), (W2, p[1]), (WL, p[2])):
        assert hp.rel_l2(host(Wt), (t.detach() - lr_ * t.grad).numpy()) <= tol


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
def test_gradient_descent_for_a_list_of_tensors(pkg, gpu, dt):
    """ptl_gradient_descent_*_multi (one launch for many structs) against the per-struct entry point."""
    nd = hp.np_dtype(dt)
    dims = [(5,), (300, 7), (1,), (64, 3, 3, 3), (1000,)] * 13  # 65 structs, 98 tensors: more than one table
    res = []
    for multi in (False, True):
        structs, keep, tensors = [], [], []
        for i, shp in enumerate(dims):
            w, g = dev(hp.uniform(0x7F00 + i, shp).astype(nd)), dev(hp.uniform(0x7F80 + i, shp).astype(nd))
            b = gb = None
            if i % 2:
                b, gb = dev(hp.uniform(0x7F40 + i, (shp[0],)).astype(nd)), dev(hp.uniform(0x7FC0 + i, (shp[0],)).astype(nd))
            o, k = hp.optim_args(pkg, dt, w, g, b, gb, 0.05, 0.01 if i % 3 == 0 else 0.0)
            structs.append(o), keep.append(k), tensors.append((w, g, b, gb))
        if multi:
            table = (type(structs[0]) * len(structs))(*structs)
            assert getattr(gpu, "ptl_gradient_descent_%s_multi" % dt)(ctypes.byref(table), len(structs)) == 0
        else:
            for o in structs:
                assert getattr(gpu, "ptl_gradient_descent_" + dt)(ctypes.byref(o)) == 0
        gpu.ptl_sync()
        res.append([[None if t is None else host(t) for t in ts] for ts in tensors])
    for one, many in zip(*res):
        for u, v in zip(one, many):
            assert (u is None and v is None) or np.array_equal(u, v)


@pytest.mark.parametrize("dt", ["fp16", "fp32"])
def test_pool_linear_loss_in_one_call(pkg, gpu, dt):
    """ptl_pool_linear_loss_*_batched against the six calls it stands for (pooling, classifier and cross-entropy forward,
    then their backward passes): the pooled vector bit for bit (same order of additions), everything behind the
    classifier's dot products to rounding - logits, loss, the gradients of logits, pooled vector and input, and the
    classifier's weight gradient after the flush of the batch it was deferred to.  Cases the one launch does not take
    (a bias, a pooling window smaller than the plane, no batch) run the six calls and give their bits."""
    import torch
    tdt = torch.float16 if dt == "fp16" else torch.float32
    tol = 2e-3 if dt == "fp16" else 1e-5
    buf = torch.empty(4 << 20, dtype=torch.uint8, device="cuda")
    #        ns, C, H, classes, bias, window, batch given, one launch expected
    cases = [(128, 64, 8, 10, 0, 8, 1, True), (7, 40, 5, 3, 0, 5, 1, True), (33, 96, 4, 32, 0, 4, 1, True),
             (16, 64, 8, 10, 1, 8, 1, False), (16, 64, 8, 10, 0, 4, 1, False), (16, 64, 8, 10, 0, 8, 0, False)]
    for case in cases:
        ns, C, H, ncls, bias, win, with_batch, expect = case
        Ho = H // win
        g = torch.Generator(device="cuda").manual_seed(ns * 1000 + C)
        x = (torch.rand(ns, C, H, H, device="cuda", generator=g) - 0.3).to(tdt)
        w = ((torch.rand(ncls, C * Ho * Ho, device="cuda", generator=g) - 0.5) * 0.5).to(tdt)
        b = (torch.rand(ncls, device="cuda", generator=g) - 0.5).to(tdt)
        target = torch.zeros(ns, ncls, device="cuda", dtype=tdt)
        target[torch.arange(ns), (3 * torch.arange(ns)) % ncls] = 1
        res = []
        for one_call in (False, True):
            dx = torch.full_like(x, 3)
            pooled, dpooled = torch.full((ns, C * Ho * Ho), 3.0, device="cuda", dtype=tdt), torch.full((ns, C * Ho * Ho), 3.0, device="cuda", dtype=tdt)
            logits, dlogits = torch.full((ns, ncls), 3.0, device="cuda", dtype=tdt), torch.full((ns, ncls), 3.0, device="cuda", dtype=tdt)
            loss, dw, db = torch.full((ns,), 3.0, device="cuda", dtype=tdt), torch.full_like(w, 3), torch.full_like(b, 3)
            pa, k1 = hp.pool_args(pkg, x, dx, pooled, dpooled, C, H, H, Ho, Ho, win, win, win, win)
            la, k2 = hp.linear_args(pkg, pooled, dpooled, w, dw, logits, dlogits, C * Ho * Ho, ncls, b if bias else None, db if bias else None)
            ca, k3 = hp.loss_args(pkg, logits, dlogits, target, loss, ncls)
            batch = pkg.WgBatch()
            batch.buf, batch.bytes = buf.data_ptr(), buf.numel()
            if one_call:
                rc = getattr(gpu, "ptl_pool_linear_loss_%s_batched" % dt)(ctypes.byref(pa), ctypes.byref(la), ctypes.byref(ca), ns,
                                                                         ctypes.byref(batch) if with_batch else None)
                assert rc == 0, gpu.ptl_last_error()
                took = batch.count == 1
                assert getattr(gpu, "ptl_conv2d_%s_wg_flush" % dt)(ctypes.byref(batch)) == 0
            else:
                for name, a, extra in (("ptl_avgpool_%s_batched", pa, (ns, 0)), ("ptl_linear_%s_fw_batched", la, (ns,)),
                                       ("ptl_cross_entropy_%s_batched", ca, (ns, 0)), ("ptl_cross_entropy_%s_batched", ca, (ns, 1)),
                                       ("ptl_linear_%s_bw_batched", la, (ns,)), ("ptl_avgpool_%s_batched", pa, (ns, 1))):
                    assert getattr(gpu, name % dt)(ctypes.byref(a), *extra) == 0, gpu.ptl_last_error()
            assert gpu.ptl_sync() == 0
            res.append((pooled, logits, loss, dlogits, dw, dpooled, dx, db))
        A, B = res
        assert took == expect, case
        names = ("pooled", "logits", "loss", "dlogits", "dw", "dpooled", "dx", "db")
        if not took:
            for i, nm in enumerate(names):
                assert torch.equal(A[i], B[i]), (case, nm)
            continue
        assert torch.equal(A[0], B[0]), case
        for i, nm in list(enumerate(names))[1:7]:
            assert hp.rel_l2(B[i].float().cpu().numpy(), A[i].float().cpu().numpy()) <= tol, (case, nm)
        assert not bool((B[6] == 3).any()) and not bool((B[4] == 3).all())
