"""Pins the CPU oracle (oracle/ptl_oracle.c) before anything is compared with it.

Each check is against something the oracle's code did not produce: a library
routine (numpy.matmul / transpose / pad, torch conv2d + autograd in float64)
on the closed-form inputs of the reference's own tests
(tests/test_matmul/utils/GM.py:81-99, tests/test_conv2d_fp32/utils/GM.py:250-263
and :306-316, tests/test_linear_fp32/utils/GM.py:78-99,
tests/test_transpose/utils/GM.py:30-48, tests/test_im2col/net.c:68-84) and on
seeded random inputs, a brute-force loop on tiny shapes, or an identity the
mathematics fixes (adjointness, involution, route equality).
"""
import ctypes

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import helpers as hp
from helpers import rel_l2

F64 = torch.float64


def t64(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64))


# ----------------------------------------------------------------------------- mm
def run_mm(pkg, orc, dt, A, B, N, M, K, tb, C0=None):
    C = np.zeros((N, M), hp.np_dtype(dt)) if C0 is None else C0
    a = hp.mm_args(pkg, A, B, C, N, M, K, tb)
    orc.call("orc_mm", dt, a)
    return C


@pytest.mark.parametrize("tb", [0, 1])
@pytest.mark.parametrize("shape", [(32, 32, 32), (24, 40, 56)])
def test_mm_reference_closed_form(pkg, orc, tb, shape):
    N, K, M = shape
    div = 1e8
    i, j = np.meshgrid(np.arange(N), np.arange(K), indexing="ij")
    A = ((1.0 + (i + j + 0.1)) / div).astype(np.float32)
    bs = (M, K) if tb else (K, M)
    i, j = np.meshgrid(np.arange(bs[0]), np.arange(bs[1]), indexing="ij")
    B = (i * j + 0.1).astype(np.float32)
    C = run_mm(pkg, orc, "fp32", A, B, N, M, K, tb)
    ref = A.astype(np.float64) @ (B.T if tb else B).astype(np.float64)
    assert rel_l2(C, ref) < 1e-6


@pytest.mark.parametrize("dt,tol", [("fp32", 2e-6), ("fp16", 6e-3)])
@pytest.mark.parametrize("N,M,K", [(1, 1, 1), (7, 5, 3), (1, 33, 20), (33, 1, 20), (9, 11, 1), (16, 24, 128)])
def test_mm_random_vs_numpy(pkg, orc, dt, tol, N, M, K):
    for tb in (0, 1):
        A = hp.normal(11 + N, (N, K), 1.0 / np.sqrt(K), hp.np_dtype(dt))
        B = hp.uniform(13 + M, (M, K) if tb else (K, M), dtype=hp.np_dtype(dt))
        C = run_mm(pkg, orc, dt, A, B, N, M, K, tb)
        ref = A.astype(np.float64) @ (B.T if tb else B).astype(np.float64)
        assert rel_l2(C, ref) < tol


def test_mm_k0_leaves_output_untouched(pkg, orc):
    C = np.full((3, 4), 5.0, np.float32)
    A = np.zeros((3, 1), np.float32)
    B = np.zeros((1, 4), np.float32)
    run_mm(pkg, orc, "fp32", A, B, 3, 4, 0, 0, C0=C)
    assert np.all(C == 5.0)


def test_mm_fp16_accumulation_sequence(pkg, orc):
    """fp16 mm keeps a half accumulator updated in k order: re-evaluate that definition in numpy."""
    N, M, K = 5, 6, 40
    A = hp.uniform(1, (N, K), dtype=np.float16)
    B = hp.uniform(2, (K, M), dtype=np.float16)
    C = run_mm(pkg, orc, "fp16", A, B, N, M, K, 0)
    ref = np.zeros((N, M), np.float16)
    for i in range(N):
        for j in range(M):
            acc = np.float16(0)
            for k in range(K):
                acc = np.float16(np.float32(acc) + np.float32(A[i, k]) * np.float32(B[k, j]))
            ref[i, j] = acc
    assert np.array_equal(C.view(np.uint16), ref.view(np.uint16))
    # and a half accumulator is visibly not a float accumulator on a long sum
    A = np.full((1, 4096), 0.25, np.float16)
    B = np.full((4096, 1), 0.25, np.float16)
    C = run_mm(pkg, orc, "fp16", A, B, 1, 1, 4096, 0)
    assert float(C[0, 0]) < 4096 * 0.0625  # stalls once the increment drops below half an ulp


# -------------------------------------------------------------------- conv2d layers
def torch_conv(x, w, pad, stride):
    """Textbook conv2d in float64; pad = (L, R, U, D), stride = (h, w). x: [N,Ci,H,W]."""
    return F.conv2d(F.pad(x, pad), w, stride=stride)


def conv_case(pkg, orc, dt, Ci, H, W, Co, Hk, Wk, pad, stride, hwc, ns=1, seed=1, bias=False):
    L, R, U, D = pad
    Ho, Wo = hp.conv_out(H, Hk, U, D, stride[0]), hp.conv_out(W, Wk, L, R, stride[1])
    nd = hp.np_dtype(dt)
    x = hp.uniform(seed, (ns, Ci, H, W), dtype=nd)
    w = hp.uniform(seed + 1, (Co, Ci, Hk, Wk), dtype=nd)
    dy = hp.uniform(seed + 2, (ns, Co, Ho, Wo), dtype=nd)
    b = hp.uniform(seed + 3, (Co,), dtype=nd) if bias else None
    tx, tw, tdy = t64(x).requires_grad_(), t64(w).requires_grad_(), t64(dy)
    tb = t64(b).requires_grad_() if bias else None
    ty = torch_conv(tx, tw, pad, stride)
    if bias:
        ty = ty + tb.view(1, -1, 1, 1)
    ty.backward(tdy)
    # layout as the layer stores it
    if hwc:
        xs, ws, dys = x.transpose(0, 2, 3, 1).copy(), w.transpose(0, 2, 3, 1).copy(), dy.transpose(0, 2, 3, 1).copy()
    else:
        xs, ws, dys = x, w, dy
    y = np.zeros_like(dys)
    dx = np.zeros_like(xs)
    dw = np.zeros_like(ws)
    db = np.zeros((Co,), nd) if bias else None
    a, keep = hp.conv2d_args(pkg, xs, dx, ws, dw, y, dys, Ci, H, W, Co, Hk, Wk, Ho, Wo, pad, stride, hwc, 1,
                             bias=b, dbias=db)
    orc.call("orc_conv2d_fw", dt, a, ns)
    orc.call("orc_conv2d_wg", dt, a, ns)
    orc.call("orc_conv2d_ig", dt, a, ns)
    if hwc:
        y, dx, dw = y.transpose(0, 3, 1, 2), dx.transpose(0, 3, 1, 2), dw.transpose(0, 3, 1, 2)
    refs = dict(y=ty.detach().numpy(), dw=tw.grad.numpy(), dx=tx.grad.numpy())
    got = dict(y=y, dw=dw, dx=dx)
    if bias:
        refs["db"], got["db"] = tb.grad.numpy(), db
    return got, refs


@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("pad,stride,Hk,Wk", [((0, 0, 0, 0), (1, 1), 3, 3), ((1, 1, 1, 1), (1, 1), 3, 3),
                                                ((1, 1, 1, 1), (2, 2), 3, 3), ((2, 2, 2, 2), (2, 2), 5, 5),
                                                ((1, 0, 0, 2), (1, 1), 3, 2), ((0, 0, 0, 0), (1, 1), 1, 1)])
def test_conv2d_fp32_vs_torch_float64(pkg, orc, hwc, pad, stride, Hk, Wk):
    H, W = 9, 11
    if (H - Hk + pad[2] + pad[3]) % stride[0] or (W - Wk + pad[0] + pad[1]) % stride[1]:
        H, W = H + 1, W + 1 if (W - Wk + pad[0] + pad[1]) % stride[1] else W
    got, ref = conv_case(pkg, orc, "fp32", 3, H, W, 4, Hk, Wk, pad, stride, hwc, ns=2, seed=5)
    for k in ref:
        assert rel_l2(got[k], ref[k]) < 2e-6, k


def test_conv2d_fp32_bias_vs_torch(pkg, orc):
    got, ref = conv_case(pkg, orc, "fp32", 3, 8, 8, 5, 3, 3, (1, 1, 1, 1), (1, 1), 0, ns=2, seed=9, bias=True)
    for k in ref:
        assert rel_l2(got[k], ref[k]) < 2e-6, k


def test_conv2d_fp16_vs_torch_float64(pkg, orc):
    got, ref = conv_case(pkg, orc, "fp16", 4, 8, 8, 6, 3, 3, (1, 1, 1, 1), (1, 1), 0, ns=2, seed=3)
    for k in ref:
        assert rel_l2(got[k], ref[k]) < 5e-3, k


def test_conv2d_reference_test_vector(pkg, orc):
    """Closed-form input/weights/label of tests/test_conv2d_fp32 (8x8 image, 3x3, 8->8, MSE loss)."""
    Ci = Co = 8
    H = W = 8
    K = 3
    Ho = Wo = 6
    c, h, w = np.meshgrid(np.arange(Ci), np.arange(H), np.arange(W), indexing="ij")
    x = (1e-3 + (c + h - w) * (c + h + w) * 1e-5).astype(np.float32)
    o, i, hk, wk = np.meshgrid(np.arange(Co), np.arange(Ci), np.arange(K), np.arange(K), indexing="ij")
    wt = ((o + i + hk + wk) * 0.01).astype(np.float32)
    label = (1.0 + np.arange(Wo) * 1e-3).astype(np.float32)[None, None, :].repeat(Co, 0).repeat(Ho, 1)
    tx, tw = t64(x)[None].requires_grad_(), t64(wt).requires_grad_()
    ty = F.conv2d(tx, tw)
    loss = F.mse_loss(ty, t64(label)[None])
    loss.backward()
    dy_ref = (2.0 * (ty.detach()[0] - t64(label)) / label.size).numpy()

    y = np.zeros((Co, Ho, Wo), np.float32)
    dx = np.zeros_like(x)
    dw = np.zeros_like(wt)
    dy = dy_ref.astype(np.float32)
    a, keep = hp.conv2d_args(pkg, x, dx, wt, dw, y, dy, Ci, H, W, Co, K, K, Ho, Wo)
    orc.call("orc_conv2d_fw", "fp32", a, 1)
    orc.call("orc_conv2d_wg", "fp32", a, 1)
    orc.call("orc_conv2d_ig", "fp32", a, 1)
    assert rel_l2(y, ty.detach().numpy()[0]) < 1e-6
    assert rel_l2(dw, tw.grad.numpy()) < 1e-5
    assert rel_l2(dx, tx.grad.numpy()[0]) < 1e-5


@pytest.mark.parametrize("pad", [(0, 0, 0, 0), (1, 1, 1, 1)])
def test_im2col_route_equals_direct_kernels(pkg, orc, pad):
    """im2row+mm (+blocktranspose) is bit-identical to the direct kernels where the reference defines it:
    all three steps without padding, the forward step also with padding."""
    Ci, Co, H, W, K = 3, 4, 7, 6, 3
    L, R, U, D = pad
    Ho, Wo = hp.conv_out(H, K, U, D, 1), hp.conv_out(W, K, L, R, 1)
    x = hp.uniform(21, (Ci, H, W))
    wt = hp.uniform(22, (Co, Ci, K, K))
    dy = hp.uniform(23, (Co, Ho, Wo))
    res = {}
    for route in (0, 1):
        y = np.zeros((Co, Ho, Wo), np.float32)
        dx = np.zeros_like(x)
        dw = np.zeros_like(wt)
        i2c = np.zeros(max(Ho * Wo * Ci * K * K, H * W * Co * K * K), np.float32)
        bt = np.zeros(Co * Ci * K * K, np.float32)
        a, keep = hp.conv2d_args(pkg, x, dx, wt, dw, y, dy, Ci, H, W, Co, K, K, Ho, Wo, pad, i2c=i2c, bt=bt)
        steps = (0, 1, 2) if pad == (0, 0, 0, 0) else (0,)
        for s in steps:
            if route:
                orc.call("orc_conv2d_im2col_route", "fp32", a, s)
            else:
                orc.call(("orc_conv2d_fw", "orc_conv2d_wg", "orc_conv2d_ig")[s], "fp32", a, 1)
        res[route] = (y, dw, dx)
    for u, v in zip(res[0], res[1]):
        assert np.array_equal(u.view(np.uint32), v.view(np.uint32))


def test_conv2d_adjoint_identities(pkg, orc):
    """<conv(x), g> = <x, IG(g)> = <W, WG(x, g)> for any x, W, g (the three steps are mutually adjoint)."""
    got, _ = conv_case(pkg, orc, "fp32", 3, 10, 10, 5, 3, 3, (1, 1, 1, 1), (2, 2), 0, ns=1, seed=31)
    x = hp.uniform(31, (1, 3, 10, 10)).astype(np.float64)
    w = hp.uniform(32, (5, 3, 3, 3)).astype(np.float64)
    g = hp.uniform(33, got["y"].shape).astype(np.float64)
    lhs = float((got["y"].astype(np.float64) * g).sum())
    assert abs(lhs - float((x * got["dx"]).sum())) < 1e-4 * abs(lhs) + 1e-4
    assert abs(lhs - float((w * got["dw"]).sum())) < 1e-4 * abs(lhs) + 1e-4


def test_batched_weight_gradient_is_sum_of_samples(pkg, orc):
    got3, _ = conv_case(pkg, orc, "fp32", 2, 6, 6, 3, 3, 3, (1, 1, 1, 1), (1, 1), 0, ns=3, seed=41)
    x = hp.uniform(41, (3, 2, 6, 6))
    dy = hp.uniform(43, (3, 3, 6, 6))
    w = hp.uniform(42, (3, 2, 3, 3))
    acc = np.zeros_like(w, dtype=np.float64)
    for n in range(3):
        dw = np.zeros_like(w)
        a, keep = hp.conv2d_args(pkg, x[n].copy(), None, w, dw, None, dy[n].copy(), 2, 6, 6, 3, 3, 3, 6, 6,
                                 (1, 1, 1, 1))
        orc.call("orc_conv2d_wg", "fp32", a, 1)
        acc += dw
    assert rel_l2(got3["dw"], acc) < 1e-6


# ------------------------------------------------------- im2row / im2col / blocktranspose
def patch_matrix_numpy(src, Hk, Wk, pad, stride, mod, Hin, Win):
    """Brute-force patch matrix [P, C, Hk, Wk] from a CHW tensor with numpy.pad + slicing."""
    C = src.shape[0]
    if mod == 0:
        L, R, U, D = pad
        p = np.pad(src, ((0, 0), (U, D), (L, R)))
        Ht, Wt = (Hin - Hk + U + D) // stride[0] + 1, (Win - Wk + L + R) // stride[1] + 1
        out = np.zeros((Ht, Wt, C, Hk, Wk), src.dtype)
        for ho in range(Ht):
            for wo in range(Wt):
                out[ho, wo] = p[:, ho * stride[0]:ho * stride[0] + Hk, wo * stride[1]:wo * stride[1] + Wk]
        return out.reshape(Ht * Wt, C, Hk, Wk)
    p = np.pad(src, ((0, 0), (Hk - 1, Hk - 1), (Wk - 1, Wk - 1)))
    out = np.zeros((Hin, Win, C, Hk, Wk), src.dtype)
    for hi in range(Hin):
        for wi in range(Win):
            out[hi, wi] = p[:, hi:hi + Hk, wi:wi + Wk]
    return out.reshape(Hin * Win, C, Hk, Wk)


def patch_args(pkg, dt, x, dy, buf, Ci, H, W, Co, Hk, Wk, Ho, Wo, pad, stride, mod, hwc):
    bi = pkg.blob(x, None, Ci, H, W)
    bw = pkg.blob(None, None, Ci, Hk, Wk)
    bo = pkg.blob(None, dy, Co, Ho, Wo)
    a = pkg.Im2colArgs()
    a.input, a.c, a.output = hp.ptr(bi), hp.ptr(bw), hp.ptr(bo)
    a.pBuffer = pkg.addr(buf)
    a.Lpad, a.Rpad, a.Upad, a.Dpad = pad
    a.mod, a.stride_h, a.stride_w, a.HWC = mod, stride[0], stride[1], hwc
    return a, [bi, bw, bo, x, dy, buf]


PATCH_CASES = [((0, 0, 0, 0), (1, 1), 0), ((1, 1, 1, 1), (1, 1), 0), ((1, 1, 1, 1), (2, 2), 0),
               ((2, 1, 0, 1), (1, 1), 0), ((0, 0, 0, 0), (1, 1), 1)]


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("pad,stride,mod", PATCH_CASES)
def test_im2row_im2col_vs_numpy_windows(pkg, orc, dt, hwc, pad, stride, mod):
    Ci, Co, H, W, Hk, Wk = 3, 2, 7, 9, 3, 3
    if mod == 0 and ((H - Hk + pad[2] + pad[3]) % stride[0] or (W - Wk + pad[0] + pad[1]) % stride[1]):
        H += 1
        W += 1 if (W - Wk + pad[0] + pad[1]) % stride[1] else 0
    Ho, Wo = (H - Hk + 1, W - Wk + 1) if mod else (hp.conv_out(H, Hk, pad[2], pad[3], stride[0]),
                                                  hp.conv_out(W, Wk, pad[0], pad[1], stride[1]))
    nd = hp.np_dtype(dt)
    # iota payload 0.1, 0.2, ... as in the reference's print-only im2col test
    x = (0.1 * (np.arange(Ci * H * W) + 1)).reshape(Ci, H, W).astype(nd)
    dy = (0.1 * (np.arange(Co * Ho * Wo) + 1)).reshape(Co, Ho, Wo).astype(nd)
    src = dy if mod else x
    ref = patch_matrix_numpy(src, Hk, Wk, pad, stride, mod, H, W)  # [P, C, Hk, Wk]
    if hwc:
        ref = ref.transpose(0, 2, 3, 1)
        xs, dys = x.transpose(1, 2, 0).copy(), dy.transpose(1, 2, 0).copy()
    else:
        xs, dys = x, dy
    P = ref.shape[0]
    ref = ref.reshape(P, -1)
    for fn, expect in (("orc_im2row", ref), ("orc_im2col", ref.T)):
        buf = np.full(ref.size, -1, nd)
        a, keep = patch_args(pkg, dt, xs, dys, buf, Ci, H, W, Co, Hk, Wk, Ho, Wo, pad, stride, mod, hwc)
        orc.call(fn, dt, a)
        assert np.array_equal(buf.reshape(expect.shape), expect), fn


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
def test_blocktranspose(pkg, orc, dt):
    Ci, Co, Hk, Wk = 3, 5, 3, 2
    nd = hp.np_dtype(dt)
    w = np.arange(Co * Ci * Hk * Wk).astype(nd)

    def bt(weights, cin, cout, hwc):
        out = np.zeros_like(weights)
        a = pkg.BlocktranspArgs()
        a.weights, a.bt_weights = pkg.addr(weights), pkg.addr(out)
        a.Cin, a.Cout, a.Hk, a.Wk, a.HWC = cin, cout, Hk, Wk, hwc
        orc.call("orc_blocktransp", dt, a)
        return out

    got = bt(w, Ci, Co, 0)
    ref = w.reshape(Co, Ci, Hk * Wk)[:, :, ::-1].transpose(1, 0, 2).reshape(-1)
    assert np.array_equal(got, ref)
    assert np.array_equal(bt(got, Co, Ci, 0), w)  # involution with the channel roles swapped
    got = bt(w, Ci, Co, 1)
    ref = w.reshape(Co, Hk, Wk, Ci)[:, ::-1, ::-1, :].transpose(3, 1, 2, 0).reshape(-1)
    assert np.array_equal(got, ref)


# --------------------------------------------------------------- transposes / layout / pad
@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("dims,axes", [((3, 4), (1, 0)), ((2, 3, 4), (2, 0, 1)), ((2, 3, 4, 5), (3, 1, 0, 2)),
                                       ((4, 1, 3), (0, 2, 1)), ((6,), (0,))])
def test_transpose_vs_numpy(pkg, orc, dt, dims, axes):
    np.random.seed(42)  # the reference's test seeds numpy with 42
    m = np.random.rand(*dims).astype(hp.np_dtype(dt))
    out = np.zeros(m.size, m.dtype)
    d = (ctypes.c_int * len(dims))(*dims)
    ax = (ctypes.c_int * len(dims))(*axes)
    a = pkg.TranspArgs()
    a.in_matrix, a.out_matrix = pkg.addr(m), pkg.addr(out)
    a.dim, a.transposed_axes, a.n_dim = d, ax, len(dims)
    orc.call("orc_transpose", dt, a)
    assert np.array_equal(out, np.transpose(m, axes).reshape(-1))


def test_transpose_matrix_and_layout_change(pkg, orc):
    m = hp.uniform(3, (5, 7))
    out = np.zeros(35, np.float32)
    a = pkg.TranspArgs()
    a.in_matrix, a.out_matrix, a.N, a.M = pkg.addr(m), pkg.addr(out), 5, 7
    orc.call("orc_transpose_matrix", "fp32", a)
    assert np.array_equal(out.reshape(7, 5), m.T)

    C, H, W = 3, 4, 5
    t = hp.uniform(4, (C, H, W))
    orig = t.copy()
    g = hp.uniform(5, (C, H, W))
    buf = np.zeros(C * H * W, np.float32)
    b = pkg.blob(t, g, C, H, W)
    la = pkg.LayoutArgs()
    la.tensor, la.transp_buffer, la.transpose_data, la.transpose_grad = hp.ptr(b), pkg.addr(buf), 1, 0
    orc.call("orc_CHW_to_HWC", "fp32", la)
    assert np.array_equal(t.reshape(H, W, C), orig.transpose(1, 2, 0))
    orc.call("orc_HWC_to_CHW", "fp32", la)
    assert np.array_equal(t, orig)  # round trip


@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("pads", [(1, 1, 1, 1), (0, 2, 1, 0), (3, 0, 0, 2)])
def test_pad_tensor_vs_numpy(pkg, orc, hwc, pads):
    L, R, U, D = pads
    C, H, W = 3, 4, 5
    x = hp.uniform(8, (C, H, W))
    ref = np.pad(x, ((0, 0), (U, D), (L, R)))
    src = x.transpose(1, 2, 0).copy() if hwc else x
    out = np.full(ref.size, -1, np.float32)
    a = pkg.PadArgs()
    a.source, a.dest, a.C, a.H, a.W = pkg.addr(src), pkg.addr(out), C, H, W
    a.T_LPAD, a.T_RPAD, a.T_UPAD, a.T_DPAD, a.HWC_lay = L, R, U, D, hwc
    orc.call("orc_pad_tensor", "fp32", a)
    expect = ref.transpose(1, 2, 0) if hwc else ref
    assert np.array_equal(out.reshape(expect.shape), expect)


# ------------------------------------------------------------------ pointwise / depthwise
@pytest.mark.parametrize("dt,tol", [("fp32", 2e-6), ("fp16", 5e-3)])
@pytest.mark.parametrize("hwc", [0, 1])
def test_pointwise_vs_numpy(pkg, orc, dt, tol, hwc):
    Ci, Co, H, W, ns = 6, 10, 5, 4, 2
    nd = hp.np_dtype(dt)
    x = hp.uniform(51, (ns, Ci, H * W), dtype=nd)
    w = hp.uniform(52, (Co, Ci), dtype=nd)
    dy = hp.uniform(53, (ns, Co, H * W), dtype=nd)
    x64, w64, dy64 = (v.astype(np.float64) for v in (x, w, dy))
    y_ref = np.einsum("oc,ncp->nop", w64, x64)
    dw_ref = np.einsum("nop,ncp->oc", dy64, x64)
    dx_ref = np.einsum("oc,nop->ncp", w64, dy64)
    if hwc:
        xs, dys = x.transpose(0, 2, 1).copy(), dy.transpose(0, 2, 1).copy()
        ws = w.T.copy() if dt == "fp32" else w  # fp32 HWC weights are [Ci][Co]
    else:
        xs, dys, ws = x, dy, w
    y, dx, dw = np.zeros_like(dys), np.zeros_like(xs), np.zeros_like(ws)
    a, keep = hp.pw_args(pkg, xs, dx, ws, dw, y, dys, Ci, Co, H, W, hwc)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_conv_pw_" + s, dt, a, ns)
    if hwc:
        y, dx = y.transpose(0, 2, 1), dx.transpose(0, 2, 1)
        dw = dw.T if dt == "fp32" else dw
    assert rel_l2(y, y_ref) < tol
    assert rel_l2(dw, dw_ref) < tol
    assert rel_l2(dx, dx_ref) < tol


@pytest.mark.parametrize("dt,pad,stride,tol", [("fp32", (0, 0, 0, 0), (1, 1), 2e-6), ("fp32", (1, 1, 1, 1), (1, 1), 2e-6),
                                               ("fp32", (1, 1, 1, 1), (2, 2), 2e-6), ("fp16", (0, 0, 0, 0), (1, 1), 5e-3)])
def test_depthwise_vs_torch_grouped_conv(pkg, orc, dt, pad, stride, tol):
    C, H, W, K, ns = 4, 9, 9, 3, 2
    L, R, U, D = pad
    Ho, Wo = hp.conv_out(H, K, U, D, stride[0]), hp.conv_out(W, K, L, R, stride[1])
    nd = hp.np_dtype(dt)
    x = hp.uniform(61, (ns, C, H, W), dtype=nd)
    w = hp.uniform(62, (C, 1, K, K), dtype=nd)
    dy = hp.uniform(63, (ns, C, Ho, Wo), dtype=nd)
    tx, tw = t64(x).requires_grad_(), t64(w).requires_grad_()
    ty = F.conv2d(F.pad(tx, pad), tw, stride=stride, groups=C)
    ty.backward(t64(dy))
    y, dx, dw = np.zeros_like(dy), np.zeros_like(x), np.zeros_like(w)
    a, keep = hp.dw_args(pkg, dt, x, dx, w, dw, y, dy, C, H, W, K, K, Ho, Wo, pad, stride)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_conv_dw_" + s, dt, a, ns)
    assert rel_l2(y, ty.detach().numpy()) < tol
    assert rel_l2(dw, tw.grad.numpy()) < tol
    assert rel_l2(dx, tx.grad.numpy()) < tol


# ------------------------------------------------------------------------------ linear
def test_linear_reference_closed_form(pkg, orc):
    """Closed-form vectors of tests/test_linear_fp32: W = 0.01, 0.02, ... row-major, label 1, MSE loss."""
    n_in, n_out = 16, 8
    x = np.full((n_in,), 1e-1, np.float32) + 0.01 * np.arange(n_in, dtype=np.float32)
    w = (0.01 * (np.arange(n_in * n_out) + 1)).reshape(n_out, n_in).astype(np.float32)
    y_ref = w.astype(np.float64) @ x.astype(np.float64)
    dy = (2.0 / n_out * (y_ref - 1.0)).astype(np.float32)
    y, dx, dw = np.zeros(n_out, np.float32), np.zeros_like(x), np.zeros_like(w)
    a, keep = hp.linear_args(pkg, x, dx, w, dw, y, dy, n_in, n_out)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_linear_" + s, "fp32", a, 1)
    assert rel_l2(y, y_ref) < 1e-6
    assert rel_l2(dw, np.outer(dy.astype(np.float64), x.astype(np.float64))) < 1e-6
    assert rel_l2(dx, dy.astype(np.float64) @ w.astype(np.float64)) < 1e-6


@pytest.mark.parametrize("dt,tol", [("fp32", 2e-6), ("fp16", 6e-3)])
def test_linear_batched_with_bias(pkg, orc, dt, tol):
    n_in, n_out, ns = 40, 24, 5
    nd = hp.np_dtype(dt)
    x = hp.normal(71, (ns, n_in), 1.0, nd)
    w = hp.normal(72, (n_out, n_in), 1.0 / np.sqrt(n_in), nd)
    b = hp.uniform(73, (n_out,), dtype=nd)
    dy = hp.uniform(74, (ns, n_out), dtype=nd)
    x64, w64, dy64 = (v.astype(np.float64) for v in (x, w, dy))
    y, dx, dw, db = np.zeros_like(dy), np.zeros_like(x), np.zeros_like(w), np.zeros_like(b)
    a, keep = hp.linear_args(pkg, x, dx, w, dw, y, dy, n_in, n_out, bias=b, dbias=db)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_linear_" + s, dt, a, ns)
    assert rel_l2(y, x64 @ w64.T + b.astype(np.float64)) < tol
    assert rel_l2(dw, dy64.T @ x64) < tol
    assert rel_l2(dx, dy64 @ w64) < tol
    assert rel_l2(db, dy64.sum(0)) < tol
