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


# ------------------------------------------------------------------ BASELINE config 4: attention step, batch 32
def mhsa_device_step(pkg, gpu, d, dy, ns, L, E, F, heads, named=False):
    """Forward and backward on device tensors, the backward reading the forward state the library itself wrote.
    Returns (forward tensors, gradients) as numpy arrays."""
    import ctypes
    sh = hp.mhsa_shapes(ns, L, E, F, heads)
    mk = lambda z: torch.from_numpy(np.ascontiguousarray(z)).to(DEV)
    data = {n: mk(v) for n, v in d.items()}
    for n in ("q", "k", "v", "p", "att", "y"):
        data[n] = mk(np.full(sh[n], 7.0, np.float32))
    diff = {n: mk(np.full(sh[n], 7.0, np.float32)) for n in ("q", "k", "v", "att", "p", "wo")}
    for n in ("wq", "wk", "wv"):
        diff[n] = mk(np.full((F, E), 7.0, np.float32))
    diff["x"] = mk(np.zeros(sh["x"], np.float32))  # the step adds to it
    diff["y"] = mk(dy)
    a, keep = hp.mhsa_args(pkg, data, diff, L, E, F, heads)
    if named:
        gpu.pulp_mhsa_fp32_fw_cl(ctypes.byref(a))
        assert gpu.ptl_last_status() == 0, gpu.ptl_last_error().decode()
        gpu.pulp_mhsa_fp32_bw_cl(ctypes.byref(a))
        assert gpu.ptl_last_status() == 0, gpu.ptl_last_error().decode()
    else:
        assert gpu.ptl_mhsa_fp32_fw_batched(ctypes.byref(a), ns) == 0, gpu.ptl_last_error().decode()
        assert gpu.ptl_mhsa_fp32_bw_batched(ctypes.byref(a), ns) == 0, gpu.ptl_last_error().decode()
    sync(gpu)
    return ({n: data[n].cpu().numpy() for n in ("q", "k", "v", "p", "att", "y")},
            {n: diff[n].cpu().numpy() for n in ("wo", "att", "p", "q", "k", "v", "wq", "wk", "wv", "x")})


def test_mhsa_config4_full_batch(pkg, orc, gpu):
    """BASELINE config 4 at its full batch: L=197, E=192, 3 heads of 64, 32 samples.  Samples of the batch equal the
    single-sample reference-named entry points bit for bit, two of them are checked against the CPU oracle, and
    the weight gradients are additive over a split of the batch."""
    import ctypes
    ns, L, E, F, heads = 32, 197, 192, 192, 3
    d, dy = hp.mhsa_inputs(0xC0DE0404, ns, L, E, F, heads)
    full_d, full_g = mhsa_device_step(pkg, gpu, d, dy, ns, L, E, F, heads)
    acts, grads = ("q", "k", "v", "p", "att", "y"), ("att", "p", "q", "k", "v", "x")
    for b in (0, 17, 31):
        db = dict(d)
        db["x"] = d["x"][b:b + 1]
        one_d, one_g = mhsa_device_step(pkg, gpu, db, dy[b:b + 1], 1, L, E, F, heads, named=True)
        for n in acts:
            assert np.array_equal(one_d[n][0], full_d[n][b]), (b, n)
        for n in grads:
            assert np.array_equal(one_g[n][0], full_g[n][b]), (b, n)
    # the CPU oracle on two samples of the batch (forward, and backward from its own forward state)
    for b in (5, 30):
        sh = hp.mhsa_shapes(1, L, E, F, heads)
        data = {n: np.ascontiguousarray(v) for n, v in d.items()}
        data["x"] = np.ascontiguousarray(d["x"][b:b + 1])
        for n in acts:
            data[n] = np.zeros(sh[n], np.float32)
        diff = {n: np.zeros(sh[n], np.float32) for n in ("q", "k", "v", "att", "p", "wo", "x")}
        for n in ("wq", "wk", "wv"):
            diff[n] = np.zeros((F, E), np.float32)
        diff["y"] = np.ascontiguousarray(dy[b:b + 1])
        a, keep = hp.mhsa_args(pkg, data, diff, L, E, F, heads)
        orc.load().orc_mhsa_fw_fp32(ctypes.byref(a), 1)
        orc.load().orc_mhsa_bw_fp32(ctypes.byref(a), 1)
        for n in acts:
            assert hp.rel_l2(full_d[n][b], data[n][0]) <= 1e-4, (b, n)
        for n in grads:
            assert hp.rel_l2(full_g[n][b], diff[n][0]) <= 1e-4, (b, n)
    # weight gradients: additive over a 12 / 20 split of the batch
    parts = []
    for lo, hi in ((0, 12), (12, 32)):
        db = dict(d)
        db["x"] = d["x"][lo:hi]
        _, g = mhsa_device_step(pkg, gpu, db, dy[lo:hi], hi - lo, L, E, F, heads)
        parts.append(g)
    for n in ("wo", "wq", "wk", "wv"):
        tot = parts[0][n].astype(np.float64) + parts[1][n].astype(np.float64)
        assert hp.rel_l2(full_g[n], tot) <= 1e-5, n


# ------------------------------------------------------------------ BASELINE config 5: ResNet-20 step, batch 128
def _resnet_inputs(ns, seed):
    x = hp.normal(seed, (ns, 3, 32, 32)).astype(np.float16)
    tgt = np.zeros((ns, 10), np.float16)
    tgt[np.arange(ns), (7 * np.arange(ns) + 3) % 10] = 1
    return x, tgt


def test_resnet20_config5_full_batch_per_sample_and_additivity(pkg, gpu):
    """ResNet-20 step, fp16, batch 128, without normalisation layers (they couple the samples): the first samples
    equal a batch of four run on its own, and the weight gradients of the batch are the sum over a 48 / 80 split."""
    import resnet_step as rs
    ns = 128
    w = rs.init_weights(0x2E600, "fp16")
    x, tgt = _resnet_inputs(ns, 0x2E601)

    def run(lo, hi):
        net = rs.ResNetStep(pkg, gpu, torch, "fp16", hi - lo, w, 0.01)
        net.x.copy_(torch.from_numpy(x[lo:hi]))
        net.target.copy_(torch.from_numpy(tgt[lo:hi]))
        net.step(update=False)
        sync(gpu)
        return net

    full = run(0, ns)
    assert torch.isfinite(full.loss).all()
    small = run(0, 4)
    # forward of a sample does not depend on its batch (kernel routes differ with the batch size: rounding only)
    assert hp.rel_l2(small.logits.cpu().numpy(), full.logits[:4].cpu().numpy()) <= 2e-3
    assert hp.rel_l2(small.loss.cpu().numpy(), full.loss[:4].cpu().numpy()) <= 2e-3
    # so does the gradient that reaches the first block
    l0 = full.conv_layers[1]
    s0 = small.conv_layers[1]
    assert l0["name"] == "s0b0c1"
    assert hp.rel_l2(s0["dx"].cpu().numpy(), l0["dx"][:4].cpu().numpy()) <= 5e-3
    a, b = run(0, 48), run(48, ns)
    for n in ("fc", "s2b2c2", "s2b0sc", "s1b0c1", "s0b0c1", "stem"):
        tot = a.dW[n].double() + b.dW[n].double()
        err = float((tot - full.dW[n].double()).norm() / full.dW[n].double().norm())
        assert err <= 5e-3, (n, err)


def test_resnet20_config5_full_batch_layer_error_budget(pkg, orc, gpu):
    """ResNet-20 step with batch normalisation, fp16, batch 128 (BASELINE config 5): every convolution,
    normalisation and classifier call is re-evaluated from the tensors THAT call read, in float64 by torch on the
    GPU, and must agree within 1e-3 (every result is an fp32 sum rounded to fp16 once: measured 2.1e-4 to 2.7e-4
    for every kind of call, forward and backward).  The end-to-end
    distance to a float64 run of the whole step is then the accumulation of these per-call roundings over the 20
    layers; it is asserted at the tolerance the small-batch test uses.  Three convolutions (the stem, a strided
    3x3 layer, a strided projection) are checked against the CPU oracle in fp32 on the same fp16 tensors."""
    import torch.nn.functional as F
    import resnet_step as rs
    from test_gpu_resnet import torch_step
    ns = 128
    w = rs.init_weights(0x2E610, "fp16")
    x, tgt = _resnet_inputs(ns, 0x2E611)
    net = rs.ResNetStep(pkg, gpu, torch, "fp16", ns, w, 0.01, norm=True)
    net.x.copy_(torch.from_numpy(x))
    net.target.copy_(torch.from_numpy(tgt))
    net.step(update=False)
    sync(gpu)
    rel = lambda got, ref: float((got.double() - ref).norm() / ref.norm())
    worst = {}
    for l in net.conv_layers:
        xd, wd, dyd = l["x"].double(), l["w"].double(), l["dy"].double()
        ref_y = F.conv2d(xd, wd, stride=l["stride"], padding=l["pad"])
        ref_dw = torch.nn.grad.conv2d_weight(xd, wd.shape, dyd, stride=l["stride"], padding=l["pad"])
        errs = {"y": rel(l["y"], ref_y), "dw": rel(l["dw"], ref_dw)}
        if l["dx"] is not None:
            ref_dx = torch.nn.grad.conv2d_input(xd.shape, wd, dyd, stride=l["stride"], padding=l["pad"])
            if "dx_extra" in l:  # the block's shortcut has added its gradient to the same buffer since
                ref_dx = ref_dx + l["dx_extra"].double()
            errs["dx"] = rel(l["dx"], ref_dx)
        for k, e in errs.items():
            assert e <= 1e-3, (l["name"], k, e)
            worst["conv " + k] = max(worst.get("conv " + k, 0.0), e)
    for l in net.norm_layers:
        xd = l["x"].double().requires_grad_(True)
        g, b = l["g"].double().requires_grad_(True), l["b"].double().requires_grad_(True)
        ref_y = F.batch_norm(xd, None, None, g, b, training=True, eps=float(np.float16(1e-5)))
        ref_y.backward(l["dy"].double())
        for k, got, ref in (("y", l["y"], ref_y.detach()), ("dx", l["dx"], xd.grad), ("dg", l["dg"], g.grad),
                            ("db", l["db"], b.grad)):
            e = rel(got, ref)
            assert e <= 1e-3, (l["name"], k, e)
            worst["norm " + k] = max(worst.get("norm " + k, 0.0), e)
    # classifier: logits = pooled W^T, dW = dlogits^T pooled, dpooled = dlogits W
    pd, wd, dl = net.pooled.double(), net.W["fc"].double(), net.dlogits.double()
    for k, got, ref in (("y", net.logits, pd @ wd.t()), ("dw", net.dW["fc"], dl.t() @ pd), ("dx", net.dpooled, dl @ wd)):
        e = rel(got, ref)
        assert e <= 1e-3, ("fc", k, e)
        worst["fc " + k] = max(worst.get("fc " + k, 0.0), e)
    print("worst per-call relative L2 errors at batch 128:", {k: "%.2e" % v for k, v in sorted(worst.items())})

    # the CPU oracle (fp32 arithmetic on the same fp16 tensors) on three convolutions of the batch
    by_name = {l["name"]: l for l in net.conv_layers}
    for name in ("stem", "s1b0c1", "s1b0sc"):
        l = by_name[name]
        xs, ws, dys = (l[k].float().cpu().numpy() for k in ("x", "w", "dy"))
        Co, Ci, K, _ = ws.shape
        H, Ho = xs.shape[2], dys.shape[2]
        p, s = l["pad"], l["stride"]
        y, dw, dx = np.zeros(dys.shape, np.float32), np.zeros_like(ws), np.zeros_like(xs)
        a, keep = hp.conv2d_args(pkg, xs, dx, ws, dw, y, dys, Ci, H, H, Co, K, K, Ho, Ho, (p, p, p, p), (s, s), 0, 0)
        steps = ("fw", "wg") + (("ig",) if l["dx"] is not None else ())
        for st in steps:
            orc.call("orc_conv2d_" + st, "fp32", a, ns)
        assert hp.rel_l2(l["y"].float().cpu().numpy(), y) <= 1e-3, name
        assert hp.rel_l2(l["dw"].float().cpu().numpy(), dw) <= 1e-3, name
        if l["dx"] is not None:
            ref = dx + (l["dx_extra"].float().cpu().numpy() if "dx_extra" in l else 0.0)
            assert hp.rel_l2(l["dx"].float().cpu().numpy(), ref) <= 1e-3, name

    # end to end against float64 (activations rounded to fp16 where the library stores them)
    ref_logits, ref_loss, ref_grads, _ = torch_step(w, x, tgt, 0.01, norm=True, stored=torch.float16, device=DEV)
    assert hp.rel_l2(net.logits.cpu().numpy(), ref_logits) <= 1.5e-1
    assert hp.rel_l2(net.loss.cpu().numpy(), ref_loss) <= 1.5e-1
    for n in ("fc", "s2b2c2", "s1b0c1", "stem"):
        assert hp.rel_l2(net.dW[n].cpu().numpy(), ref_grads[n]) <= 1.5e-1, n
