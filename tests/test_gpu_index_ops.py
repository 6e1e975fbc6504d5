"""GPU parity of the index-permutation and streaming helpers: bit-exact against the CPU oracle."""
import ctypes

import numpy as np
import pytest
import torch

import helpers as hp
from test_oracle_pin import PATCH_CASES, patch_args

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32 if a.dtype == np.float32 else np.uint16)


def sync(lib):
    assert lib.ptl_sync() == 0, lib.ptl_last_error().decode()


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("pad,stride,mod", PATCH_CASES)
def test_im2row_im2col(pkg, orc, gpu, dt, hwc, pad, stride, mod):
    Ci, Co, H, W, Hk, Wk = 5, 4, 13, 11, 3, 3
    if mod == 0 and ((H - Hk + pad[2] + pad[3]) % stride[0] or (W - Wk + pad[0] + pad[1]) % stride[1]):
        H += 1
        W += 1 if (W - Wk + pad[0] + pad[1]) % stride[1] else 0
    Ho, Wo = (H - Hk + 1, W - Wk + 1) if mod else (hp.conv_out(H, Hk, pad[2], pad[3], stride[0]),
                                                  hp.conv_out(W, Wk, pad[0], pad[1], stride[1]))
    nd = hp.np_dtype(dt)
    x = hp.uniform(1, (Ci * H * W,), dtype=nd)
    dy = hp.uniform(2, (Co * Ho * Wo,), dtype=nd)
    n = (H * W * Co if mod else Ho * Wo * Ci) * Hk * Wk
    for fn in ("im2row", "im2col"):
        buf = np.full(n, -1, nd)
        a, keep = patch_args(pkg, dt, x, dy, buf, Ci, H, W, Co, Hk, Wk, Ho, Wo, pad, stride, mod, hwc)
        orc.call("orc_" + fn, dt, a)
        gx, gdy, gbuf = dev(x), dev(dy), dev(np.full(n, -2, nd))
        g, keep2 = patch_args(pkg, dt, gx, gdy, gbuf, Ci, H, W, Co, Hk, Wk, Ho, Wo, pad, stride, mod, hwc)
        pkg.call("pulp_%s_%s" % (fn, dt), g)
        sync(gpu)
        assert np.array_equal(bits(gbuf.cpu().numpy()), bits(buf)), fn


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
def test_blocktranspose(pkg, orc, gpu, dt, hwc):
    Ci, Co, Hk, Wk = 16, 32, 3, 3
    nd = hp.np_dtype(dt)
    w = hp.uniform(3, (Co * Ci * Hk * Wk,), dtype=nd)
    ref = np.zeros_like(w)
    a = pkg.BlocktranspArgs()
    a.weights, a.bt_weights, a.Cin, a.Cout, a.Hk, a.Wk, a.HWC = pkg.addr(w), pkg.addr(ref), Ci, Co, Hk, Wk, hwc
    orc.call("orc_blocktransp", dt, a)
    gw, gbt = dev(w), dev(np.zeros_like(w))
    g = pkg.BlocktranspArgs()
    g.weights, g.bt_weights, g.Cin, g.Cout, g.Hk, g.Wk, g.HWC = pkg.addr(gw), pkg.addr(gbt), Ci, Co, Hk, Wk, hwc
    pkg.call("pulp_blocktransp_" + dt, g)
    sync(gpu)
    assert np.array_equal(bits(gbt.cpu().numpy()), bits(ref))
    if not hwc:  # applying it again with the channel roles swapped restores the weights
        gback = dev(np.zeros_like(w))
        g.weights, g.bt_weights, g.Cin, g.Cout = pkg.addr(gbt), pkg.addr(gback), Co, Ci
        pkg.call("pulp_blocktransp_" + dt, g)
        sync(gpu)
        assert np.array_equal(bits(gback.cpu().numpy()), bits(w))


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("dims,axes", [((3, 4), (1, 0)), ((128, 64), (1, 0)), ((65, 130), (1, 0)),
                                       ((2, 3, 4), (2, 0, 1)), ((3, 197, 64), (0, 2, 1)), ((2, 3, 4, 5), (3, 1, 0, 2)),
                                       ((6,), (0,))])
def test_transpose(pkg, gpu, dt, dims, axes):
    np.random.seed(42)
    m = np.random.rand(*dims).astype(hp.np_dtype(dt))
    gm, gout = dev(m), dev(np.zeros(m.size, m.dtype))
    d = (ctypes.c_int * len(dims))(*dims)
    ax = (ctypes.c_int * len(dims))(*axes)
    a = pkg.TranspArgs()
    a.in_matrix, a.out_matrix, a.dim, a.transposed_axes, a.n_dim = pkg.addr(gm), pkg.addr(gout), d, ax, len(dims)
    pkg.call("transpose" if dt == "fp32" else "transpose_fp16", a)
    sync(gpu)
    assert np.array_equal(gout.cpu().numpy(), np.transpose(m, axes).reshape(-1))
    if len(dims) == 2:
        gout.zero_()
        a.N, a.M = dims
        pkg.call("transpose_matrix" if dt == "fp32" else "transpose_matrix_fp16", a)
        sync(gpu)
        assert np.array_equal(gout.cpu().numpy(), m.T.reshape(-1))


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
def test_layout_change_round_trip(pkg, gpu, dt):
    C, H, W = 16, 32, 32
    nd = hp.np_dtype(dt)
    t, gr = hp.uniform(4, (C, H, W), dtype=nd), hp.uniform(5, (C, H, W), dtype=nd)
    gt, gg, gbuf = dev(t), dev(gr), dev(np.zeros(C * H * W, nd))
    b = pkg.blob(gt, gg, C, H, W)
    la = pkg.LayoutArgs()
    la.tensor, la.transp_buffer, la.transpose_data, la.transpose_grad = hp.ptr(b), pkg.addr(gbuf), 1, 1
    sfx = "" if dt == "fp32" else "_fp16"
    pkg.call("CHW_to_HWC" + sfx, la)
    sync(gpu)
    assert np.array_equal(gt.cpu().numpy().reshape(H, W, C), t.transpose(1, 2, 0))
    assert np.array_equal(gg.cpu().numpy().reshape(H, W, C), gr.transpose(1, 2, 0))
    assert np.array_equal(gbuf.cpu().numpy().reshape(H, W, C), gr.transpose(1, 2, 0))  # buffer keeps the last result
    pkg.call("HWC_to_CHW" + sfx, la)
    sync(gpu)
    assert np.array_equal(gt.cpu().numpy(), t) and np.array_equal(gg.cpu().numpy(), gr)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("pads", [(1, 1, 1, 1), (0, 2, 1, 0)])
def test_pad_tensor(pkg, gpu, dt, hwc, pads):
    L, R, U, D = pads
    C, H, W = 5, 9, 7
    nd = hp.np_dtype(dt)
    x = hp.uniform(8, (C, H, W), dtype=nd)
    ref = np.pad(x, ((0, 0), (U, D), (L, R)))
    src = x.transpose(1, 2, 0) if hwc else x
    gs, gd = dev(src), dev(np.full(ref.size, -1, nd))
    a = pkg.PadArgs()
    a.source, a.dest, a.C, a.H, a.W = pkg.addr(gs), pkg.addr(gd), C, H, W
    a.T_LPAD, a.T_RPAD, a.T_UPAD, a.T_DPAD, a.HWC_lay = L, R, U, D, hwc
    pkg.call("pad_tensor" if dt == "fp32" else "pad_tensor_fp16", a)
    sync(gpu)
    expect = ref.transpose(1, 2, 0) if hwc else ref
    assert np.array_equal(gd.cpu().numpy().reshape(expect.shape), expect)


def test_streaming_helpers(pkg, gpu):
    n = 1000003
    x, y = hp.uniform(1, (n,)), hp.uniform(2, (n,))
    gx, gy, gz = dev(x), dev(y), dev(np.zeros(n, np.float32))
    c = pkg.CopyArgs()
    c.from_, c.to, c.size = pkg.addr(gx), pkg.addr(gz), n
    pkg.call("copy", c)
    sync(gpu)
    assert torch.equal(gz, gx)
    v = pkg.VectSumArgs()
    v.op_1, v.op_2, v.dest, v.size = pkg.addr(gx), pkg.addr(gy), pkg.addr(gz), n
    pkg.call("vect_sum", v)
    sync(gpu)
    assert np.array_equal(gz.cpu().numpy(), x + y)
    s = pkg.SetToValueArgs()
    s.to, s.value, s.size = pkg.addr(gz), 0.375, n - 3
    pkg.call("set_to_value", s)
    sync(gpu)
    out = gz.cpu().numpy()
    assert np.all(out[:n - 3] == 0.375) and np.array_equal(out[n - 3:], (x + y)[n - 3:])
    # fp16 twins and the casts
    hx, hy = x.astype(np.float16), y.astype(np.float16)
    ghx, ghy, ghz = dev(hx), dev(hy), dev(np.zeros(n, np.float16))
    v.op_1, v.op_2, v.dest = pkg.addr(ghx), pkg.addr(ghy), pkg.addr(ghz)
    pkg.call("vect_sum_fp16", v)
    sync(gpu)
    assert np.array_equal(ghz.cpu().numpy(), hx + hy)
    s16 = pkg.SetToValueArgsFp16()
    s16.to, s16.value, s16.size = pkg.addr(ghz), int(np.float16(-1.5).view(np.uint16)), 10
    pkg.call("set_to_value_fp16", s16)
    c.from_, c.to, c.size = pkg.addr(ghx), pkg.addr(ghy), n
    pkg.call("copy_fp16", c)
    sync(gpu)
    assert np.all(ghz.cpu().numpy()[:10] == np.float16(-1.5)) and torch.equal(ghy, ghx)
    k = pkg.CastArgs()
    k.source, k.destination, k.size = pkg.addr(ghx), pkg.addr(gz), n
    pkg.call("cast_fp16_tensor_to_fp32", k)
    sync(gpu)
    assert np.array_equal(gz.cpu().numpy(), hx.astype(np.float32))
    k.source, k.destination = pkg.addr(gx), pkg.addr(ghz)
    pkg.call("cast_fp32_tensor_to_fp16", k)
    sync(gpu)
    assert np.array_equal(ghz.cpu().numpy(), x.astype(np.float16))


# ---------------------------------------------------------------- larger and ragged shapes for the chunked kernels
@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("N,M", [(256, 512), (72, 200), (1000, 24), (8, 8), (136, 1048), (63, 129)])
def test_transpose_matrix_tiles(pkg, gpu, dt, N, M):
    """Whole and ragged 64x64 tiles, sizes that are and are not multiples of a 16-byte chunk."""
    nd = hp.np_dtype(dt)
    m = hp.uniform(0x7A05, (N, M), dtype=nd)
    gm, gout = dev(m), dev(np.full(N * M, 3, nd))
    a = pkg.TranspArgs()
    a.in_matrix, a.out_matrix, a.N, a.M = pkg.addr(gm), pkg.addr(gout), N, M
    pkg.call("transpose_matrix" if dt == "fp32" else "transpose_matrix_fp16", a)
    sync(gpu)
    assert np.array_equal(bits(gout.cpu().numpy()), bits(m.T.reshape(-1)))


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("Ci,Co,Hk,Wk", [(64, 96, 3, 3), (40, 33, 3, 3), (72, 64, 5, 5), (8, 16, 1, 1), (130, 70, 2, 3),
                                         (256, 320, 3, 3), (296, 264, 3, 3), (264, 256, 1, 1)])
def test_blocktranspose_tiles(pkg, orc, gpu, dt, hwc, Ci, Co, Hk, Wk):
    nd = hp.np_dtype(dt)
    w = hp.uniform(0xB7, (Co * Ci * Hk * Wk,), dtype=nd)
    ref = np.zeros_like(w)
    a = pkg.BlocktranspArgs()
    a.weights, a.bt_weights, a.Cin, a.Cout, a.Hk, a.Wk, a.HWC = pkg.addr(w), pkg.addr(ref), Ci, Co, Hk, Wk, hwc
    orc.call("orc_blocktransp", dt, a)
    gw, gbt = dev(w), dev(np.full(w.shape, 3, nd))
    g = pkg.BlocktranspArgs()
    g.weights, g.bt_weights, g.Cin, g.Cout, g.Hk, g.Wk, g.HWC = pkg.addr(gw), pkg.addr(gbt), Ci, Co, Hk, Wk, hwc
    pkg.call("pulp_blocktransp_" + dt, g)
    sync(gpu)
    assert np.array_equal(bits(gbt.cpu().numpy()), bits(ref))


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("Ci,H,W,K,pad,stride,mod", [(16, 32, 32, 3, (1, 1, 1, 1), (1, 1), 0), (7, 19, 23, 3, (1, 1, 1, 1), (2, 2), 0),
                                                     (6, 14, 9, 5, (2, 2, 2, 2), (1, 1), 0), (5, 12, 12, 3, (0, 0, 0, 0), (1, 1), 1),
                                                     (16, 32, 32, 1, (0, 0, 0, 0), (1, 1), 0), (64, 40, 48, 1, (0, 0, 0, 0), (1, 1), 0),
                                                     (8, 20, 24, 5, (2, 2, 2, 2), (1, 1), 0), (4, 19, 16, 3, (1, 1, 1, 1), (2, 1), 0),
                                                     (3, 8, 8, 3, (1, 1, 1, 1), (1, 1), 0), (6, 10, 16, 3, (0, 0, 0, 0), (1, 1), 1),
                                                     (2, 70, 136, 3, (1, 1, 1, 1), (1, 1), 0),
                                                     (5, 12, 16, 3, (0, 2, 2, 0), (1, 1), 0), (4, 11, 16, 3, (1, 1, 0, 1), (1, 1), 0),
                                                     (3, 10, 16, 7, (3, 3, 3, 3), (1, 1), 0), (5, 9, 24, 3, (1, 1, 2, 3), (1, 1), 0)])
def test_im2row_im2col_chunked(pkg, orc, gpu, dt, hwc, Ci, H, W, K, pad, stride, mod):
    """Patch matrices whose rows are not multiples of a 16-byte chunk (chunks straddle rows and columns), BASELINE
    config 1 among them; rows as wide as the image at unit strides (the column-major matrix as shifted copies of the
    planes: 3x3, 5x5 and 7x7 filters, padding on one side only, more padding above and below than the filter needs)."""
    Co = 4
    Ho, Wo = (H - K + 1, W - K + 1) if mod else (hp.conv_out(H, K, pad[2], pad[3], stride[0]),
                                                hp.conv_out(W, K, pad[0], pad[1], stride[1]))
    nd = hp.np_dtype(dt)
    x = hp.uniform(11, (Ci * H * W,), dtype=nd)
    dy = hp.uniform(12, (Co * Ho * Wo,), dtype=nd)
    n = (H * W * Co if mod else Ho * Wo * Ci) * K * K
    for fn in ("im2row", "im2col"):
        buf = np.full(n, -1, nd)
        a, keep = patch_args(pkg, dt, x, dy, buf, Ci, H, W, Co, K, K, Ho, Wo, pad, stride, mod, hwc)
        orc.call("orc_" + fn, dt, a)
        gx, gdy, gbuf = dev(x), dev(dy), dev(np.full(n, -2, nd))
        g, keep2 = patch_args(pkg, dt, gx, gdy, gbuf, Ci, H, W, Co, K, K, Ho, Wo, pad, stride, mod, hwc)
        pkg.call("pulp_%s_%s" % (fn, dt), g)
        sync(gpu)
        assert np.array_equal(bits(gbuf.cpu().numpy()), bits(buf)), fn
        # an unaligned buffer takes the element-wise kernel: same result one element further
        gbig = dev(np.full(n + 8, -2, nd))
        g.pBuffer = pkg.addr(gbig) + gbig.element_size()
        pkg.call("pulp_%s_%s" % (fn, dt), g)
        sync(gpu)
        assert np.array_equal(bits(gbig.cpu().numpy()[1:n + 1]), bits(buf)), fn


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("C,H,W,pads", [(16, 32, 32, (1, 1, 1, 1)), (5, 9, 13, (2, 0, 1, 3)), (3, 7, 7, (0, 0, 0, 0)),
                                         (64, 60, 52, (1, 1, 1, 1)), (7, 130, 37, (3, 2, 0, 5)), (2, 5, 4001, (1, 0, 1, 1)),
                                         (33, 3, 5, (0, 4, 2, 0)), (3, 700, 9, (1, 2, 300, 1))])
def test_pad_tensor_chunked(pkg, orc, gpu, dt, hwc, C, H, W, pads):
    nd = hp.np_dtype(dt)
    R, L, U, D = pads
    src = hp.uniform(21, (C * H * W,), dtype=nd)
    n = C * (H + U + D) * (W + L + R)
    ref = np.full(n, -1, nd)
    a = pkg.PadArgs()
    a.source, a.dest, a.C, a.H, a.W = pkg.addr(src), pkg.addr(ref), C, H, W
    a.T_RPAD, a.T_LPAD, a.T_UPAD, a.T_DPAD, a.HWC_lay = R, L, U, D, hwc
    orc.call("orc_pad_tensor", dt, a)
    gs, gd = dev(src), dev(np.full(n, -2, nd))
    g = pkg.PadArgs()
    g.source, g.dest, g.C, g.H, g.W = pkg.addr(gs), pkg.addr(gd), C, H, W
    g.T_RPAD, g.T_LPAD, g.T_UPAD, g.T_DPAD, g.HWC_lay = R, L, U, D, hwc
    pkg.call("pad_tensor" if dt == "fp32" else "pad_tensor_fp16", g)
    sync(gpu)
    assert np.array_equal(bits(gd.cpu().numpy()), bits(ref))


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("n", [1, 7, 8, 1000, 4099])
def test_copy_sizes(pkg, gpu, dt, n):
    nd = hp.np_dtype(dt)
    src = hp.uniform(31, (n + 4,), dtype=nd)
    for shift in (0, 1):  # aligned and unaligned source
        gs, gd = dev(src), dev(np.full(n + 4, 3, nd))
        c = pkg.CopyArgs()
        c.from_, c.to, c.size = pkg.addr(gs) + shift * gs.element_size(), pkg.addr(gd), n
        pkg.call("copy" if dt == "fp32" else "copy_fp16", c)
        sync(gpu)
        out = gd.cpu().numpy()
        assert np.array_equal(bits(out[:n]), bits(src[shift:shift + n])) and np.all(out[n:] == 3)
