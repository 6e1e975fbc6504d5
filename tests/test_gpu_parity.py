"""GPU parity: every entry point of libptl_hip.so against the CPU oracle on the same seeded inputs.

Bars (BASELINE north star): fp32 outputs and gradients within 1e-4 relative L2 of the oracle, fp16 within
1e-2 of the fp16-accumulating oracle, index work bit-exact.  All calls go through the C ABI; tensors live in
device memory (torch is only the allocator) unless a test says it passes host pointers.
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


# ------------------------------------------------------------------------------ Conv2D
def conv_parity(pkg, orc, lib, dt, Ci, H, W, Co, Hk, Wk, pad, stride, hwc, ns, seed, im2col=1, bias=False,
                host_ptrs=False, via_batched=None):
    L, R, U, D = pad
    Ho, Wo = hp.conv_out(H, Hk, U, D, stride[0]), hp.conv_out(W, Wk, L, R, stride[1])
    nd = hp.np_dtype(dt)
    xs = (ns, H, W, Ci) if hwc else (ns, Ci, H, W)
    ws = (Co, Hk, Wk, Ci) if hwc else (Co, Ci, Hk, Wk)
    ys = (ns, Ho, Wo, Co) if hwc else (ns, Co, Ho, Wo)
    x = hp.uniform(seed, xs, dtype=nd)
    w = hp.uniform(seed + 1, ws, dtype=nd)
    dy = hp.uniform(seed + 2, ys, dtype=nd)
    b = hp.uniform(seed + 3, (Co,), dtype=nd) if bias else None
    # oracle
    y, dx, dw = np.zeros(ys, nd), np.zeros(xs, nd), np.zeros(ws, nd)
    db = np.zeros((Co,), nd) if bias else None
    a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, Hk, Wk, Ho, Wo, pad, stride, hwc, im2col, b, db)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_conv2d_" + s, dt, a, ns)
    # HIP
    if host_ptrs:
        gx, gw, gdy, gb = x, w, dy, b
        gy, gdx, gdw = np.full(ys, 3, nd), np.full(xs, 3, nd), np.full(ws, 3, nd)
        gdb = np.full((Co,), 3, nd) if bias else None
    else:
        gx, gw, gdy, gb = dev(x), dev(w), dev(dy), dev(b)
        gy, gdx, gdw = dev(np.full(ys, 3, nd)), dev(np.full(xs, 3, nd)), dev(np.full(ws, 3, nd))
        gdb = dev(np.full((Co,), 3, nd)) if bias else None
    g, keep2 = hp.conv2d_args(pkg, gx, gdx, gw, gdw, gy, gdy, Ci, H, W, Co, Hk, Wk, Ho, Wo, pad, stride, hwc, im2col,
                              gb, gdb)
    if via_batched is None:
        via_batched = ns != 1
    if via_batched:
        for s in ("fw", "wg", "ig"):
            pkg.call("ptl_conv2d_%s_%s_batched" % (dt, s), g, ns)
    else:
        pkg.call("pulp_conv2d_%s_fw_cl" % dt, g)
        pkg.call("pulp_conv2d_%s_bw_cl" % dt, g)
    sync(lib)
    out = [("y", gy, y), ("dw", gdw, dw), ("dx", gdx, dx)]
    if bias:
        out.append(("db", gdb, db))
    errs = {}
    for name, got, ref in out:
        got = got if host_ptrs else host(got)
        errs[name] = rel_l2(got, ref)
        assert errs[name] <= TOL[dt], (name, errs[name])
    return errs


CONV_CASES = [
    # Ci, H, W, Co, Hk, Wk, pad(L,R,U,D), stride
    (16, 32, 32, 32, 3, 3, (1, 1, 1, 1), (1, 1)),  # BASELINE config 1
    (8, 8, 8, 8, 3, 3, (0, 0, 0, 0), (1, 1)),      # reference test default
    (3, 17, 13, 5, 3, 3, (1, 1, 1, 1), (2, 2)),
    (4, 15, 15, 6, 5, 5, (2, 2, 2, 2), (2, 2)),
    (5, 9, 12, 7, 3, 2, (1, 0, 0, 2), (1, 1)),
    (16, 12, 12, 16, 1, 1, (0, 0, 0, 0), (1, 1)),
    (3, 32, 32, 16, 3, 3, (1, 1, 1, 1), (1, 1)),   # ResNet-20 stem geometry
    (16, 33, 33, 32, 3, 3, (1, 1, 1, 1), (2, 2)),
]


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_batch1(pkg, orc, gpu, dt, hwc, case):
    Ci, H, W, Co, Hk, Wk, pad, stride = case
    conv_parity(pkg, orc, gpu, dt, Ci, H, W, Co, Hk, Wk, pad, stride, hwc, 1, 0xC0DE0001)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
def test_conv2d_batched(pkg, orc, gpu, dt, hwc):
    conv_parity(pkg, orc, gpu, dt, 16, 32, 32, 32, 3, 3, (1, 1, 1, 1), (1, 1), hwc, 5, 0xC0DE0011)
    conv_parity(pkg, orc, gpu, dt, 6, 11, 11, 9, 3, 3, (1, 1, 1, 1), (2, 2), hwc, 3, 0xC0DE0012)


# Strided single-tap layers (projection shortcuts): the input gradient is one product scattered into the zeroed
# tensor.  Outputs start as 3s, so positions the layer never read must come back as zeros.
@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("case", [(16, 11, 11, 32, (2, 2), 5), (6, 9, 13, 10, (2, 3), 3), (32, 15, 8, 64, (2, 1), 4)])
def test_conv2d_strided_single_tap(pkg, orc, gpu, dt, hwc, case):
    Ci, H, W, Co, stride, ns = case
    conv_parity(pkg, orc, gpu, dt, Ci, H, W, Co, 1, 1, (0, 0, 0, 0), stride, hwc, ns, 0xC0DE0081,
                via_batched=True)


# With bottom / right padding the last output rows and columns of such a layer sit on padded positions outside
# the input: their gradient contributions must be dropped, not scattered into the neighbouring plane.
@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("case", [(6, 5, 7, 10, (0, 2, 0, 2), (2, 2), 3), (8, 6, 6, 16, (0, 1, 0, 0), (1, 2), 2),
                                  (16, 9, 9, 32, (0, 0, 0, 2), (2, 2), 4)])
def test_conv2d_strided_single_tap_with_trailing_padding(pkg, orc, gpu, dt, hwc, case):
    Ci, H, W, Co, pad, stride, ns = case
    conv_parity(pkg, orc, gpu, dt, Ci, H, W, Co, 1, 1, pad, stride, hwc, ns, 0xC0DE0082, via_batched=True)


# The direct convolution kernel (channel-major forward and input gradient) normally takes only calls with
# many pixel tiles; selection 2 sends every call whose geometry fits through it, so that small cases the
# oracle finishes in seconds cover its tile logic: tiles that start mid-row, span several images, hang over
# the end, strides, asymmetric pads, channel counts off the MFMA step, several filter tiles.
DIRECT_CASES = [
    # Ci, H, W, Co, Hk, Wk, pad(L,R,U,D), stride, ns
    (16, 32, 32, 32, 3, 3, (1, 1, 1, 1), (1, 1), 3),
    (3, 17, 13, 5, 3, 3, (1, 1, 1, 1), (2, 2), 7),
    (4, 15, 15, 6, 5, 5, (2, 2, 2, 2), (2, 2), 5),
    (5, 9, 12, 7, 3, 2, (1, 0, 0, 2), (1, 1), 9),
    (16, 12, 12, 16, 1, 1, (0, 0, 0, 0), (1, 1), 4),
    (20, 6, 6, 40, 3, 3, (1, 1, 1, 1), (1, 1), 11),    # tiles span several images
    (33, 40, 7, 130, 3, 3, (1, 1, 1, 1), (1, 1), 2),    # narrow rows, channels off the k step, several filter tiles
    (8, 20, 70, 9, 3, 3, (0, 1, 2, 0), (1, 2), 2),      # rows wider than a wave
    (6, 11, 11, 9, 3, 3, (1, 1, 1, 1), (2, 2), 3),
    (2, 5, 5, 3, 5, 5, (2, 2, 2, 2), (1, 1), 30),       # filter as large as the image
]


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("case", DIRECT_CASES)
def test_conv2d_direct_kernel(pkg, orc, gpu, dt, case):
    Ci, H, W, Co, Hk, Wk, pad, stride, ns = case
    gpu.ptl_set_gemm_path(2)
    try:
        conv_parity(pkg, orc, gpu, dt, Ci, H, W, Co, Hk, Wk, pad, stride, 0, ns, 0xC0DE0041, via_batched=True)
        # the last call of conv_parity is the input gradient (32 filters of 130 fp32 channels and 9 taps
        # exceed LDS: GEMM route)
        assert gpu.ptl_last_conv_direct() == (0 if (Co == 130 and dt == "fp32") else 1)
        nd = hp.np_dtype(dt)
        Ho, Wo = hp.conv_out(H, Hk, pad[2], pad[3], stride[0]), hp.conv_out(W, Wk, pad[0], pad[1], stride[1])
        x, w = dev(np.zeros((ns, Ci, H, W), nd)), dev(np.zeros((Co, Ci, Hk, Wk), nd))
        y = dev(np.zeros((ns, Co, Ho, Wo), nd))
        a, keep = hp.conv2d_args(pkg, x, None, w, None, y, None, Ci, H, W, Co, Hk, Wk, Ho, Wo, pad, stride)
        pkg.call("ptl_conv2d_%s_fw_batched" % dt, a, ns)
        assert gpu.ptl_last_conv_direct() == 1
    finally:
        gpu.ptl_set_gemm_path(0)


# Channel-minor (HWC) tensors already consist of the 16-byte channel chunks the direct kernel works on:
# forward and input gradient read them in place (channel counts that are multiples of the vector).
DIRECT_HWC_CASES = [
    (16, 32, 32, 32, 3, 3, (1, 1, 1, 1), (1, 1), 3),
    (8, 9, 12, 7, 3, 2, (1, 0, 0, 2), (1, 1), 9),
    (24, 6, 6, 40, 3, 3, (1, 1, 1, 1), (1, 1), 11),
    (16, 17, 13, 12, 3, 3, (1, 1, 1, 1), (2, 2), 7),
    (40, 10, 10, 130, 1, 1, (0, 0, 0, 0), (1, 1), 4),
]


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("case", DIRECT_HWC_CASES)
def test_conv2d_direct_kernel_hwc(pkg, orc, gpu, dt, case):
    Ci, H, W, Co, Hk, Wk, pad, stride, ns = case
    gpu.ptl_set_gemm_path(2)
    try:
        conv_parity(pkg, orc, gpu, dt, Ci, H, W, Co, Hk, Wk, pad, stride, 1, ns, 0xC0DE0061, via_batched=True)
        # the last call of conv_parity is the input gradient: its input has Co channels
        vec = 8 if dt == "fp16" else 4
        assert gpu.ptl_last_conv_direct() == (1 if Co % vec == 0 else 0)
    finally:
        gpu.ptl_set_gemm_path(0)


# Unit-stride layers whose channel counts are multiples of a 128-byte slab (64 halves / 32 floats) run as a sum
# over filter taps on the look-up-free GEMM (padded, channel-blocked copy of the input): forward when Ci fits,
# input gradient when Co does.  Cases: square and ragged images, asymmetric padding, 5x5 and 2x3 filters, tile
# counts that leave a ragged last tile, channel counts of one and several slabs.
TAP_CASES = [
    # Ci, H, W, Co, Hk, Wk, pad(L,R,U,D), ns
    (64, 14, 14, 64, 3, 3, (1, 1, 1, 1), 4),
    (128, 9, 11, 64, 3, 3, (1, 1, 1, 1), 3),
    (64, 12, 10, 130, 3, 3, (0, 2, 1, 0), 2),
    (64, 8, 8, 192, 5, 5, (2, 2, 2, 2), 2),
    (192, 7, 9, 64, 2, 3, (1, 1, 0, 1), 5),
    (64, 6, 6, 64, 3, 3, (0, 0, 0, 0), 1),
]


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("case", TAP_CASES)
def test_conv2d_tap_sum_route(pkg, orc, gpu, dt, case):
    Ci, H, W, Co, Hk, Wk, pad, ns = case
    slab = 64 if dt == "fp16" else 32
    gpu.ptl_set_gemm_path(3)
    try:
        conv_parity(pkg, orc, gpu, dt, Ci, H, W, Co, Hk, Wk, pad, (1, 1), 0, ns, 0xC0DE0071, via_batched=True)
        # the last call of conv_parity is the input gradient, whose "input" channels are Co
        assert gpu.ptl_last_conv_direct() == (1 if Co % slab == 0 else 0)
        # forward and weight gradient alone: both take a convolution kernel
        nd = hp.np_dtype(dt)
        Ho, Wo = hp.conv_out(H, Hk, pad[2], pad[3], 1), hp.conv_out(W, Wk, pad[0], pad[1], 1)
        x, w = dev(hp.uniform(1, (ns, Ci, H, W), dtype=nd)), dev(hp.uniform(2, (Co, Ci, Hk, Wk), dtype=nd))
        dy = dev(hp.uniform(3, (ns, Co, Ho, Wo), dtype=nd))
        y, dw = dev(np.zeros((ns, Co, Ho, Wo), nd)), dev(np.zeros((Co, Ci, Hk, Wk), nd))
        a, keep = hp.conv2d_args(pkg, x, None, w, dw, y, dy, Ci, H, W, Co, Hk, Wk, Ho, Wo, pad, (1, 1))
        for s in ("fw", "wg"):
            pkg.call("ptl_conv2d_%s_%s_batched" % (dt, s), a, ns)
            assert gpu.ptl_last_conv_direct() == 1, s
    finally:
        gpu.ptl_set_gemm_path(0)


# 3x3 fp16 channel-major layers through the kernel that keeps the input tile in LDS for all nine taps (path 5):
# forward when Ci and Co are multiples of 64, input gradient likewise.  Cases: one and two channel slabs, 64 and
# 128 filters per tile, asymmetric padding, images small enough for the bottom rows of the padded grid to be left out
# (tiles that cross one and two sample boundaries), the widest image the tile holds, too wide an image (falls back).
RESIDENT_CASES = [
    # Ci, H, W, Co, pad(L,R,U,D), ns, resident
    (64, 14, 14, 64, (1, 1, 1, 1), 4, 1),
    (64, 28, 28, 64, (1, 1, 1, 1), 3, 1),
    (128, 9, 11, 64, (1, 1, 1, 1), 3, 1),
    (64, 12, 10, 128, (0, 2, 1, 0), 2, 1),
    (64, 7, 61, 64, (1, 1, 1, 1), 1, 1),
    (64, 5, 62, 64, (1, 1, 1, 1), 1, 1),    # the widest row whose reach (two rows of W + 1 positions + 2) fits
    (64, 5, 63, 64, (1, 1, 1, 1), 1, 0),
    (192, 6, 6, 256, (0, 0, 0, 0), 2, 1),
    (64, 3, 3, 64, (0, 0, 0, 0), 1, 1),     # one output pixel per sample, a single ragged tile
    (64, 3, 5, 128, (1, 1, 1, 1), 1, 1),
    (64, 16, 16, 64, (1, 1, 1, 1), 17, 1),  # tiles that straddle two sample boundaries with the bottom rows left out
]


# (channels in, height, width, channels between, channels out, padding of the first layer, of the second, batch)
CHAIN_CASES = [(64, 14, 14, 64, 64, (1, 1, 1, 1), (1, 1, 1, 1), 12), (64, 9, 11, 128, 64, (1, 1, 1, 1), (0, 2, 1, 1), 20),
               (128, 28, 28, 64, 128, (1, 1, 1, 1), (1, 1, 1, 1), 5), (64, 12, 10, 192, 64, (1, 1, 1, 1), (1, 1, 0, 0), 9),
               (32, 16, 16, 64, 64, (1, 1, 1, 1), (1, 1, 1, 1), 8)]


@pytest.mark.parametrize("case", CHAIN_CASES)
def test_conv2d_layers_in_a_row_hand_the_blocked_copy_on(pkg, gpu, case):
    """ptl_conv2d_fp16_fw_batched_chained: the forward kernel of a layer writes its output a second time as the padded,
    channel-blocked copy the next layer reads; the next layer's forward and weight-gradient calls take that copy
    instead of making one.  Same bits as the plain calls everywhere; the copy really is what is read (the tensor
    itself is overwritten before the second layer runs); a first layer that does not take the resident-tile route
    (32 channels) leaves the copy invalid and the second layer makes its own; with `relu` set the copy is the blocked
    form of the rectified output, for a second layer behind a ReLU."""
    Ci, H, W, Cm, Co, pad1, pad2, ns = case
    H1, W1 = H + pad1[2] + pad1[3] - 2, W + pad1[0] + pad1[1] - 2
    H2, W2 = H1 + pad2[2] + pad2[3] - 2, W1 + pad2[0] + pad2[1] - 2
    x = (torch.rand(ns, Ci, H, W, device="cuda") - 0.5).half()
    w1 = ((torch.rand(Cm, Ci, 3, 3, device="cuda") - 0.5) * 0.2).half()
    w2 = ((torch.rand(Co, Cm, 3, 3, device="cuda") - 0.5) * 0.2).half()
    dy2 = (torch.rand(ns, Co, H2, W2, device="cuda") - 0.5).half()
    gpu.ptl_set_gemm_path(5)
    try:
        # plain calls
        y1, y2, dw2 = torch.full((ns, Cm, H1, W1), 3.0, device="cuda").half(), torch.full_like(dy2, 3), torch.full_like(w2, 3)
        a1, k1 = hp.conv2d_args(pkg, x, None, w1, None, y1, None, Ci, H, W, Cm, 3, 3, H1, W1, pad1, (1, 1))
        a2, k2 = hp.conv2d_args(pkg, y1, None, w2, dw2, y2, dy2, Cm, H1, W1, Co, 3, 3, H2, W2, pad2, (1, 1))
        pkg.call("ptl_conv2d_fp16_fw_batched", a1, ns)
        pkg.call("ptl_conv2d_fp16_fw_batched", a2, ns)
        pkg.call("ptl_conv2d_fp16_wg_batched", a2, ns)
        gpu.ptl_sync()
        # the same two layers with the copy handed on
        z1, z2, ew2 = torch.full_like(y1, 5), torch.full_like(dy2, 5), torch.full_like(w2, 5)
        b1, k3 = hp.conv2d_args(pkg, x, None, w1, None, z1, None, Ci, H, W, Cm, 3, 3, H1, W1, pad1, (1, 1))
        b2, k4 = hp.conv2d_args(pkg, z1, None, w2, ew2, z2, dy2, Cm, H1, W1, Co, 3, 3, H2, W2, pad2, (1, 1))
        nbytes = gpu.ptl_conv2d_fp16_cache_bytes(ctypes.byref(b2), ns)
        assert nbytes > 0
        buf = torch.full((nbytes,), 0x3c, dtype=torch.uint8, device="cuda")
        c = pkg.ConvCache()
        c.buf, c.bytes = buf.data_ptr(), nbytes
        assert gpu.ptl_conv2d_fp16_cache_prepare(ctypes.byref(b2), ns, ctypes.byref(c)) == 0
        assert gpu.ptl_conv2d_fp16_fw_batched_chained(ctypes.byref(b1), ns, None, ctypes.byref(c)) == 0
        handed_on = Ci % 64 == 0
        assert c.valid == (1 if handed_on else 0)
        gpu.ptl_sync()
        assert torch.equal(z1, y1)
        if handed_on:
            # the copy is the second layer's padded, blocked input: [Cm/8][ns][Hp][Wp][8] with zero halo
            Hp, Wp = H1 + max(pad2[2], pad2[3]), W1 + max(pad2[0], pad2[1])
            blk = buf[:Cm // 8 * ns * Hp * Wp * 16].view(torch.float16).view(Cm // 8, ns, Hp, Wp, 8)
            want = torch.zeros_like(blk)
            want[:, :, pad2[2]:pad2[2] + H1, pad2[0]:pad2[0] + W1, :] = y1.view(ns, Cm // 8, 8, H1, W1).permute(1, 0, 3, 4, 2)
            assert torch.equal(blk, want)
            assert int(buf[Cm // 8 * ns * Hp * Wp * 16:].max()) == 0
            z1.fill_(7)  # what the second layer must NOT read
        assert gpu.ptl_conv2d_fp16_fw_batched_chained(ctypes.byref(b2), ns, ctypes.byref(c), None) == 0
        assert gpu.ptl_last_conv_resident() == 1
        assert c.valid == 1  # (handed on, or filled by this call)
        assert gpu.ptl_conv2d_fp16_wg_batched_cached(ctypes.byref(b2), ns, ctypes.byref(c)) == 0
        gpu.ptl_sync()
        assert torch.equal(z2, y2)
        if handed_on and gpu.ptl_last_conv_resident() == 1:  # (the weight-gradient route that reads the copy)
            assert torch.equal(ew2, dw2)
        elif not handed_on:
            assert torch.equal(ew2, dw2)
        # a cache of another geometry is not read
        if handed_on:
            z1.copy_(y1)
            c.geometry[2] += 1
            z3 = torch.full_like(dy2, 5)
            b3, k5 = hp.conv2d_args(pkg, z1, None, w2, None, z3, None, Cm, H1, W1, Co, 3, 3, H2, W2, pad2, (1, 1))
            buf.fill_(0x3c)
            assert gpu.ptl_conv2d_fp16_fw_batched_chained(ctypes.byref(b3), ns, ctypes.byref(c), None) == 0
            gpu.ptl_sync()
            assert torch.equal(z3, y2)
        # behind a ReLU: the copy holds max(output, 0), i.e. the blocked form of the activation's output
        if handed_on:
            c2 = pkg.ConvCache()
            c2.buf, c2.bytes, c2.relu = buf.data_ptr(), nbytes, 1
            r1 = torch.relu(y1)
            z4, z5 = torch.full_like(y1, 5), torch.full_like(dy2, 5)
            b4, k7 = hp.conv2d_args(pkg, x, None, w1, None, z4, None, Ci, H, W, Cm, 3, 3, H1, W1, pad1, (1, 1))
            b5, k8 = hp.conv2d_args(pkg, r1, None, w2, None, z5, None, Cm, H1, W1, Co, 3, 3, H2, W2, pad2, (1, 1))
            y5 = torch.full_like(dy2, 3)
            a5r, k9 = hp.conv2d_args(pkg, r1, None, w2, None, y5, None, Cm, H1, W1, Co, 3, 3, H2, W2, pad2, (1, 1))
            pkg.call("ptl_conv2d_fp16_fw_batched", a5r, ns)
            assert gpu.ptl_conv2d_fp16_cache_prepare(ctypes.byref(b5), ns, ctypes.byref(c2)) == 0
            assert gpu.ptl_conv2d_fp16_fw_batched_chained(ctypes.byref(b4), ns, None, ctypes.byref(c2)) == 0
            assert c2.valid == 1
            gpu.ptl_sync()
            assert torch.equal(z4, y1)  # the layer's own output is not rectified
            Hp, Wp = H1 + max(pad2[2], pad2[3]), W1 + max(pad2[0], pad2[1])
            blk = buf[:Cm // 8 * ns * Hp * Wp * 16].view(torch.float16).view(Cm // 8, ns, Hp, Wp, 8)
            want = torch.zeros_like(blk)
            want[:, :, pad2[2]:pad2[2] + H1, pad2[0]:pad2[0] + W1, :] = r1.view(ns, Cm // 8, 8, H1, W1).permute(1, 0, 3, 4, 2)
            assert torch.equal(blk, want)
            keep_r1 = r1.clone()
            r1.fill_(7)
            assert gpu.ptl_conv2d_fp16_fw_batched_chained(ctypes.byref(b5), ns, ctypes.byref(c2), None) == 0
            gpu.ptl_sync()
            assert torch.equal(z5, y5)
            r1.copy_(keep_r1)
        # a producing layer with a bias writes no copy (the bias is added behind its kernel)
        if handed_on:
            bias = (torch.rand(Cm, device="cuda") - 0.5).half()
            z6 = torch.full_like(y1, 5)
            b6, k10 = hp.conv2d_args(pkg, x, None, w1, None, z6, None, Ci, H, W, Cm, 3, 3, H1, W1, pad1, (1, 1), bias=bias)
            c3 = pkg.ConvCache()
            c3.buf, c3.bytes = buf.data_ptr(), nbytes
            assert gpu.ptl_conv2d_fp16_cache_prepare(ctypes.byref(b2), ns, ctypes.byref(c3)) == 0
            assert gpu.ptl_conv2d_fp16_fw_batched_chained(ctypes.byref(b6), ns, None, ctypes.byref(c3)) == 0
            gpu.ptl_sync()
            assert c3.valid == 0
            assert float((z6.float() - (y1.float() + bias.float().view(1, Cm, 1, 1))).abs().max()) <= 2e-2
        # a reader that would not use a copy: prepare says so
        small = torch.zeros(ns, 32, 8, 8, device="cuda").half()
        ws = torch.zeros(64, 32, 3, 3, device="cuda").half()
        ys = torch.zeros(ns, 64, 8, 8, device="cuda").half()
        a5, k6 = hp.conv2d_args(pkg, small, None, ws, None, ys, None, 32, 8, 8, 64, 3, 3, 8, 8, (1, 1, 1, 1), (1, 1))
        assert gpu.ptl_conv2d_fp16_cache_prepare(ctypes.byref(a5), ns, ctypes.byref(c)) == 1
    finally:
        gpu.ptl_set_gemm_path(0)


@pytest.mark.parametrize("case", [(64, 14, 14, 64, (1, 1, 1, 1), 12), (128, 9, 11, 64, (0, 2, 1, 1), 20),
                                  (64, 28, 28, 128, (1, 1, 1, 1), 5), (32, 16, 16, 64, (1, 1, 1, 1), 8)])
def test_conv2d_forward_leaves_its_blocked_input_for_the_gradients(pkg, gpu, case):
    """ptl_conv2d_fp16_*_cached: the forward call fills the caller's buffer with its padded, channel-blocked copy of
    the input, the weight-gradient and the weight + input-gradient calls read it - same results, bit for bit, as the
    plain calls; a layer that does not build such a copy (32 channels) leaves the cache invalid and the calls fall
    back; a cache of another geometry is ignored."""
    Ci, H, W, Co, pad, ns = case
    pl, pr, pu, pd = pad
    Ho, Wo = H + pu + pd - 2, W + pl + pr - 2
    x = (torch.rand(ns, Ci, H, W, device="cuda") - 0.5).half()
    w = ((torch.rand(Co, Ci, 3, 3, device="cuda") - 0.5) * 0.2).half()
    dy = (torch.rand(ns, Co, Ho, Wo, device="cuda") - 0.5).half()
    outs = []
    for cached in (False, True):
        y, dx, dw, dw2 = torch.full_like(dy, 3), torch.full_like(x, 3), torch.full_like(w, 3), torch.full_like(w, 3)
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, pad, (1, 1))
        a2, keep2 = hp.conv2d_args(pkg, x, None, w, dw2, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, pad, (1, 1))
        gpu.ptl_set_gemm_path(5)
        try:
            if cached:
                nbytes = gpu.ptl_conv2d_fp16_cache_bytes(ctypes.byref(a), ns)
                assert (nbytes > 0) == (Ci % 64 == 0)
                buf = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
                c = pkg.ConvCache()
                c.buf, c.bytes = buf.data_ptr(), nbytes
                assert gpu.ptl_conv2d_fp16_fw_batched_cached(ctypes.byref(a), ns, ctypes.byref(c)) == 0
                assert c.valid == (1 if Ci % 64 == 0 else 0)
                assert gpu.ptl_conv2d_fp16_bw_batched_cached(ctypes.byref(a), ns, ctypes.byref(c)) == 0
                assert gpu.ptl_conv2d_fp16_wg_batched_cached(ctypes.byref(a2), ns, ctypes.byref(c)) == 0
                if c.valid:  # a copy of another layer's geometry must not be used
                    other = pkg.ConvCache()
                    other.buf, other.bytes, other.valid = buf.data_ptr(), nbytes, 1
                    for i, v in enumerate((ns, Ci, H + pu + pd + 1, W + pl + pr, pu, pl)):
                        other.geometry[i] = v
                    buf.fill_(0x3c)
                    dw3 = torch.full_like(w, 3)
                    a3, keep3 = hp.conv2d_args(pkg, x, None, w, dw3, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, pad, (1, 1))
                    assert gpu.ptl_conv2d_fp16_wg_batched_cached(ctypes.byref(a3), ns, ctypes.byref(other)) == 0
                    gpu.ptl_sync()
                    assert torch.equal(dw3, dw2)
                    # ... and a valid cache IS what the resident-tile weight gradient reads: with every chunk of the
                    # copy (border included) overwritten by 0x3c3c = 1.05859375, each filter's gradient is that constant
                    # times the sum of its output gradient, whatever the tap and channel
                    dw4 = torch.full_like(w, 3)
                    a4, keep4 = hp.conv2d_args(pkg, x, None, w, dw4, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, pad, (1, 1))
                    assert gpu.ptl_conv2d_fp16_wg_batched_cached(ctypes.byref(a4), ns, ctypes.byref(c)) == 0
                    took_copy = gpu.ptl_last_conv_resident() == 1  # (the route that reads the copy: 128-filter tiles)
                    gpu.ptl_sync()
                    assert took_copy == (Co % 128 == 0)
                    if took_copy:
                        want = (1.05859375 * dy.float().sum(dim=(0, 2, 3))).view(Co, 1, 1, 1).expand_as(w)
                        assert float((dw4.float() - want).norm() / want.norm()) <= 2e-3
                    else:
                        assert torch.equal(dw4, dw2)
            else:
                pkg.call("ptl_conv2d_fp16_fw_batched", a, ns)
                pkg.call("ptl_conv2d_fp16_bw_batched", a, ns)
                pkg.call("ptl_conv2d_fp16_wg_batched", a2, ns)
        finally:
            gpu.ptl_set_gemm_path(0)
        gpu.ptl_sync()
        outs.append((y, dx, dw, dw2))
    for plain, kept in zip(*outs):
        assert torch.equal(plain, kept)
    ref_dw = torch.nn.grad.conv2d_weight(torch.nn.functional.pad(x.float(), pad), w.shape, dy.float())
    assert float((outs[1][3].float() - ref_dw).norm() / ref_dw.norm()) <= 2e-3


@pytest.mark.parametrize("case", RESIDENT_CASES)
def test_conv2d_resident_tile_route(pkg, orc, gpu, case):
    Ci, H, W, Co, pad, ns, resident = case
    gpu.ptl_set_gemm_path(5)
    try:
        conv_parity(pkg, orc, gpu, "fp16", Ci, H, W, Co, 3, 3, pad, (1, 1), 0, ns, 0xC0DE0075, via_batched=True)
        assert gpu.ptl_last_conv_resident() == resident  # (the input gradient ran last)
    finally:
        gpu.ptl_set_gemm_path(0)


@pytest.mark.parametrize("case", [(64, 12, 10, 128, (0, 2, 1, 0), 2), (192, 6, 6, 256, (0, 0, 0, 0), 2),
                                  (128, 14, 14, 128, (1, 1, 1, 1), 9), (64, 3, 3, 128, (0, 0, 0, 0), 1),
                                  (64, 5, 61, 128, (1, 1, 1, 1), 3)])
def test_conv2d_resident_tile_weight_gradient(pkg, orc, gpu, case):
    """The weight gradient on the channel-blocked layouts (path 5; filters a multiple of 128, channels of 64):
    against the oracle; ragged last unit, one and several channel tiles."""
    Ci, H, W, Co, pad, ns = case
    nd = np.float16
    Ho, Wo = hp.conv_out(H, 3, pad[2], pad[3], 1), hp.conv_out(W, 3, pad[0], pad[1], 1)
    x, w = hp.uniform(31, (ns, Ci, H, W), dtype=nd), hp.uniform(32, (Co, Ci, 3, 3), dtype=nd)
    dy = hp.uniform(33, (ns, Co, Ho, Wo), dtype=nd)
    ref = np.zeros((Co, Ci, 3, 3), nd)
    a, keep = hp.conv2d_args(pkg, x, None, w, ref, np.zeros((ns, Co, Ho, Wo), nd), dy, Ci, H, W, Co, 3, 3, Ho, Wo, pad, (1, 1))
    orc.call("orc_conv2d_wg", "fp16", a, ns)
    gdw = dev(np.full((Co, Ci, 3, 3), 3, nd))
    g, keep2 = hp.conv2d_args(pkg, dev(x), None, dev(w), gdw, dev(np.zeros((ns, Co, Ho, Wo), nd)), dev(dy), Ci, H, W, Co,
                              3, 3, Ho, Wo, pad, (1, 1))
    gpu.ptl_set_gemm_path(5)
    try:
        pkg.call("ptl_conv2d_fp16_wg_batched", g, ns)
        assert gpu.ptl_last_conv_resident() == 1
    finally:
        gpu.ptl_set_gemm_path(0)
    sync(gpu)
    assert rel_l2(host(gdw), ref) <= TOL["fp16"]


@pytest.mark.parametrize("case", [(128, 14, 14, 128, (1, 1, 1, 1), 9, 1), (64, 12, 10, 128, (0, 2, 1, 1), 7, 1),
                                  (64, 12, 10, 128, (1, 1, 1, 1), 7, 1), (16, 9, 9, 8, (1, 1, 1, 1), 3, 0),
                                  (64, 12, 10, 128, (0, 0, 0, 0), 7, 0)])
@pytest.mark.parametrize("skip", [(0, 0), (1, 0), (0, 1)])
def test_conv2d_backward_in_one_call(pkg, orc, gpu, case, skip):
    """ptl_conv2d_fp16_bw_batched against the oracle's two steps: layers that share the blocked copy of the output
    gradient between the resident-tile kernels (symmetric and asymmetric "same" padding), layers that fall back to
    the two single steps, and the skip flags (a skipped gradient must stay untouched)."""
    Ci, H, W, Co, pad, ns, shared = case
    nd = np.float16
    Ho, Wo = hp.conv_out(H, 3, pad[2], pad[3], 1), hp.conv_out(W, 3, pad[0], pad[1], 1)
    x, w = hp.uniform(41, (ns, Ci, H, W), dtype=nd), hp.uniform(42, (Co, Ci, 3, 3), dtype=nd)
    dy = hp.uniform(43, (ns, Co, Ho, Wo), dtype=nd)
    rdw, rdx = np.zeros((Co, Ci, 3, 3), nd), np.zeros((ns, Ci, H, W), nd)
    a, keep = hp.conv2d_args(pkg, x, rdx, w, rdw, np.zeros((ns, Co, Ho, Wo), nd), dy, Ci, H, W, Co, 3, 3, Ho, Wo, pad, (1, 1))
    orc.call("orc_conv2d_wg", "fp16", a, ns)
    orc.call("orc_conv2d_ig", "fp16", a, ns)
    gdw, gdx = dev(np.full((Co, Ci, 3, 3), 3, nd)), dev(np.full((ns, Ci, H, W), 3, nd))
    g, keep2 = hp.conv2d_args(pkg, dev(x), gdx, dev(w), gdw, dev(np.zeros((ns, Co, Ho, Wo), nd)), dev(dy), Ci, H, W, Co,
                              3, 3, Ho, Wo, pad, (1, 1))
    g.skip_wg_grad, g.skip_in_grad = skip
    gpu.ptl_set_gemm_path(5 if shared else 0)
    try:
        pkg.call("ptl_conv2d_fp16_bw_batched", g, ns)
        if skip == (0, 0):
            assert gpu.ptl_last_conv_resident() == shared
    finally:
        gpu.ptl_set_gemm_path(0)
    sync(gpu)
    if skip[0]:
        assert np.all(host(gdw) == 3)
    else:
        assert rel_l2(host(gdw), rdw) <= TOL["fp16"]
    if skip[1]:
        assert np.all(host(gdx) == 3)
    else:
        assert rel_l2(host(gdx), rdx) <= TOL["fp16"]


@pytest.mark.parametrize("case", [(64, 14, 14, 128, 9), (128, 5, 7, 64, 21), (64, 62, 62, 64, 2), (192, 28, 28, 256, 5),
                                  (64, 3, 61, 128, 4), (128, 1, 1, 128, 300), (64, 30, 9, 192, 3)])
def test_conv2d_resident_tile_channel_minor_in_place(pkg, gpu, case):
    """Channel-minor 3x3 "same" layers on the resident-tile kernel that reads X[b][y][x][c] in place (the zero border
    comes from the addresses of its loads): forward and input gradient against torch in float32; tiles that cross
    several samples, a single row, the widest row that fits, ragged last tiles, one and several filter tiles and
    channel slabs."""
    import torch.nn.functional as F
    Ci, H, W, Co, ns = case
    nd = np.float16
    x = dev(hp.uniform(51, (ns, H, W, Ci), dtype=nd))
    w = dev(hp.uniform(52, (Co, 3, 3, Ci), dtype=nd) * 0.2)
    dy = dev(hp.uniform(53, (ns, H, W, Co), dtype=nd))
    y, dx = dev(np.full((ns, H, W, Co), 3, nd)), dev(np.full((ns, H, W, Ci), 3, nd))
    a, keep = hp.conv2d_args(pkg, x, dx, w, None, y, dy, Ci, H, W, Co, 3, 3, H, W, (1, 1, 1, 1), (1, 1), 1)
    gpu.ptl_set_gemm_path(5)
    try:
        for s in ("fw", "ig"):
            pkg.call("ptl_conv2d_fp16_%s_batched" % s, a, ns)
            assert gpu.ptl_last_conv_resident() == 1, s
    finally:
        gpu.ptl_set_gemm_path(0)
    sync(gpu)
    xc, wc, dyc = x.float().permute(0, 3, 1, 2), w.float().permute(0, 3, 1, 2), dy.float().permute(0, 3, 1, 2)
    ref_y = F.conv2d(xc, wc, padding=1).permute(0, 2, 3, 1)
    ref_dx = torch.nn.grad.conv2d_input(xc.shape, wc, dyc, padding=1).permute(0, 2, 3, 1)
    rel = lambda got, ref: float((got.float() - ref).norm() / ref.norm())
    assert rel(y, ref_y) <= 1e-3
    assert rel(dx, ref_dx) <= 1e-3


@pytest.mark.parametrize("case", [(64, 14, 14, 128, 9), (128, 5, 7, 128, 21), (64, 62, 62, 128, 2), (192, 28, 28, 256, 5),
                                  (64, 3, 61, 128, 4), (128, 1, 1, 128, 300), (64, 30, 9, 384, 3),
                                  (64, 14, 14, 64, 9), (128, 5, 7, 192, 21), (64, 62, 62, 64, 2), (64, 1, 1, 64, 300),
                                  (192, 20, 20, 320, 7)])
def test_conv2d_resident_tile_weight_gradient_channel_minor_in_place(pkg, gpu, case):
    """The resident-tile weight gradient on channel-minor tensors read in place (128-filter tiles in two tap groups;
    64-filter tiles with all nine taps where the filters are no multiple of 128): against torch in float32 and against
    the tap-sum route; the filter gradient is [Cout][3][3][Cin].  Units that cross several samples, a single row,
    the widest row that fits, a ragged last unit, several filter and channel tiles."""
    Ci, H, W, Co, ns = case
    nd = np.float16
    x = dev(hp.uniform(61, (ns, H, W, Ci), dtype=nd))
    w = dev(hp.uniform(62, (Co, 3, 3, Ci), dtype=nd) * 0.2)
    dy = dev(hp.uniform(63, (ns, H, W, Co), dtype=nd))
    res = {}
    for path in (5, 3):
        dw, y = dev(np.full((Co, 3, 3, Ci), 3, nd)), dev(np.zeros((ns, H, W, Co), nd))
        a, keep = hp.conv2d_args(pkg, x, None, w, dw, y, dy, Ci, H, W, Co, 3, 3, H, W, (1, 1, 1, 1), (1, 1), 1)
        gpu.ptl_set_gemm_path(path)
        try:
            pkg.call("ptl_conv2d_fp16_wg_batched", a, ns)
            assert gpu.ptl_last_conv_resident() == (1 if path == 5 else 0)
        finally:
            gpu.ptl_set_gemm_path(0)
        sync(gpu)
        res[path] = dw
    xc, dyc = x.float().permute(0, 3, 1, 2), dy.float().permute(0, 3, 1, 2)
    ref = torch.nn.grad.conv2d_weight(xc, (Co, Ci, 3, 3), dyc, padding=1).permute(0, 2, 3, 1)
    rel = lambda got, r: float((got.float() - r).norm() / r.norm())
    assert rel(res[5], ref) <= 1e-3
    assert rel(res[5], res[3].float()) <= 2e-3
    # both gradients in one call (the reference's pulp_conv2d_fp16_bw_cl pattern) take the same two kernels
    dw, dx, y = dev(np.full((Co, 3, 3, Ci), 3, nd)), dev(np.full((ns, H, W, Ci), 3, nd)), dev(np.zeros((ns, H, W, Co), nd))
    a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, 3, 3, H, W, (1, 1, 1, 1), (1, 1), 1)
    gpu.ptl_set_gemm_path(5)
    try:
        pkg.call("ptl_conv2d_fp16_bw_batched", a, ns)
    finally:
        gpu.ptl_set_gemm_path(0)
    sync(gpu)
    assert torch.equal(dw, res[5])
    ref_dx = torch.nn.grad.conv2d_input(xc.shape, w.float().permute(0, 3, 1, 2), dyc, padding=1).permute(0, 2, 3, 1)
    assert rel(dx, ref_dx) <= 1e-3


@pytest.mark.parametrize("case", [(64, 32, 14, 14, 9), (128, 96, 10, 12, 5), (64, 32, 56, 56, 3), (192, 160, 7, 30, 4)])
def test_conv2d_resident_tile_32_filter_tiles(pkg, gpu, case):
    """Filter counts that are multiples of 32 but not of 64 on the resident-tile kernel (32-filter tiles): the forward
    pass of a layer into such a count and the input gradient of the mirrored layer (channel-major), against torch
    in float32."""
    import torch.nn.functional as F
    Ci, Co, H, W, ns = case
    nd = np.float16
    rel = lambda got, ref: float((got.float() - ref).norm() / ref.norm())
    x = dev(hp.uniform(71, (ns, Ci, H, W), dtype=nd))
    w = dev(hp.uniform(72, (Co, Ci, 3, 3), dtype=nd) * 0.2)
    y = dev(np.full((ns, Co, H, W), 3, nd))
    a, keep = hp.conv2d_args(pkg, x, None, w, None, y, None, Ci, H, W, Co, 3, 3, H, W, (1, 1, 1, 1), (1, 1))
    # mirrored layer Co -> Ci: its input gradient is a convolution from Ci channels to Co filters
    w2 = dev(hp.uniform(73, (Ci, Co, 3, 3), dtype=nd) * 0.2)
    dy2 = dev(hp.uniform(74, (ns, Ci, H, W), dtype=nd))
    dx2, x2 = dev(np.full((ns, Co, H, W), 3, nd)), dev(np.zeros((ns, Co, H, W), nd))
    b, keep2 = hp.conv2d_args(pkg, x2, dx2, w2, None, None, dy2, Co, H, W, Ci, 3, 3, H, W, (1, 1, 1, 1), (1, 1))
    gpu.ptl_set_gemm_path(5)
    try:
        pkg.call("ptl_conv2d_fp16_fw_batched", a, ns)
        assert gpu.ptl_last_conv_resident() == 1
        pkg.call("ptl_conv2d_fp16_ig_batched", b, ns)
        assert gpu.ptl_last_conv_resident() == 1
    finally:
        gpu.ptl_set_gemm_path(0)
    sync(gpu)
    assert rel(y, F.conv2d(x.float(), w.float(), padding=1)) <= 1e-3
    assert rel(dx2, torch.nn.grad.conv2d_input((ns, Co, H, W), w2.float(), dy2.float(), padding=1)) <= 1e-3


def test_conv2d_resident_tile_many_tiles(pkg, gpu):
    """More position tiles than workgroups (every workgroup walks several tiles, the last one ragged) and two
    filter tiles: the resident-tile kernel against the tap-sum GEMM and against torch in float32."""
    import torch.nn.functional as F
    Ci, Co, H, W, ns = 128, 256, 30, 30, 80
    nd = np.float16
    x, w = dev(hp.uniform(21, (ns, Ci, H, W), dtype=nd)), dev(hp.uniform(22, (Co, Ci, 3, 3), dtype=nd) * 0.1)
    dy = dev(hp.uniform(23, (ns, Co, H, W), dtype=nd))
    res = {}
    for path in (3, 5):
        y, dx = dev(np.zeros((ns, Co, H, W), nd)), dev(np.zeros((ns, Ci, H, W), nd))
        dw = dev(np.zeros((Co, Ci, 3, 3), nd))
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, 3, 3, H, W, (1, 1, 1, 1), (1, 1))
        gpu.ptl_set_gemm_path(path)
        try:
            for s in ("fw", "ig", "wg"):
                pkg.call("ptl_conv2d_fp16_%s_batched" % s, a, ns)
                assert gpu.ptl_last_conv_resident() == (1 if path == 5 else 0), s
        finally:
            gpu.ptl_set_gemm_path(0)
        sync(gpu)
        res[path] = [y.float(), dx.float(), dw.float()]
    ref_y = F.conv2d(x.float(), w.float(), padding=1)
    ref_dx = torch.nn.grad.conv2d_input(x.shape, w.float(), dy.float(), padding=1)
    ref_dw = torch.nn.grad.conv2d_weight(x.float(), w.shape, dy.float(), padding=1)
    rel = lambda got, ref: float((got - ref).norm() / ref.norm())
    for got, other, ref in zip(res[5], res[3], (ref_y, ref_dx, ref_dw)):
        assert rel(got, ref) <= 1e-3
        assert rel(got, other) <= 1e-3


def test_conv2d_routes_agree_on_large_channels(pkg, gpu):
    """The tap-sum route, the direct kernels and the implicit-im2col GEMM give the same forward, weight gradient
    and input gradient (fp16, 64 -> 64 channels)."""
    Ci = Co = 64
    H = W = 14
    ns = 6
    nd = np.float16
    x, w = dev(hp.uniform(11, (ns, Ci, H, W), dtype=nd)), dev(hp.uniform(12, (Co, Ci, 3, 3), dtype=nd))
    dy = dev(hp.uniform(13, (ns, Co, H, W), dtype=nd))
    res = {}
    for path in (1, 2, 3):
        y, dx, dw = (dev(np.zeros(s, nd)) for s in ((ns, Co, H, W), (ns, Ci, H, W), (Co, Ci, 3, 3)))
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, 3, 3, H, W, (1, 1, 1, 1), (1, 1))
        gpu.ptl_set_gemm_path(path)
        try:
            for s in ("fw", "wg", "ig"):
                pkg.call("ptl_conv2d_fp16_%s_batched" % s, a, ns)
        finally:
            gpu.ptl_set_gemm_path(0)
        sync(gpu)
        res[path] = [host(t).astype(np.float64) for t in (y, dw, dx)]
    for path in (2, 3):
        for got, ref in zip(res[path], res[1]):
            assert rel_l2(got, ref) <= 2e-3


# The direct weight-gradient kernel needs unit column stride and row lengths that are multiples of the
# 16-byte vector (8 halves / 4 floats).
DIRECT_WG_CASES = [
    # Ci, H, W, Co, Hk, Wk, pad(L,R,U,D), stride, ns
    (16, 32, 32, 32, 3, 3, (1, 1, 1, 1), (1, 1), 3),
    (5, 9, 16, 7, 3, 3, (1, 1, 1, 1), (2, 1), 6),       # row stride 2
    (20, 6, 8, 40, 3, 3, (1, 1, 1, 1), (1, 1), 11),     # tiles span several images; two channel slabs
    (33, 12, 24, 70, 3, 3, (1, 1, 1, 1), (1, 1), 2),    # two channel slabs, two row tiles
    (12, 12, 24, 70, 5, 3, (1, 1, 2, 2), (1, 1), 2),    # 15 taps
    (8, 10, 8, 9, 1, 1, (0, 0, 0, 0), (1, 1), 5),       # single tap
    (3, 9, 40, 4, 3, 5, (2, 2, 0, 2), (1, 1), 2),       # pads on three sides, 5 columns of taps
    (4, 3, 128, 6, 3, 3, (1, 1, 1, 1), (1, 1), 2),      # one output row per tile
    (9, 8, 16, 5, 3, 3, (2, 0, 1, 1), (1, 1), 3),       # all the column padding on the left
    (9, 8, 16, 5, 3, 3, (0, 2, 1, 1), (1, 1), 3),       # ... on the right
    (40, 8, 8, 33, 3, 3, (1, 1, 1, 1), (1, 1), 5),      # a tile is a whole sample
    (96, 8, 8, 96, 3, 3, (1, 1, 1, 1), (1, 1), 2),      # large filter tensor, two partial sums (vector reduction)
]


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("case", DIRECT_WG_CASES)
def test_conv2d_direct_weight_gradient(pkg, orc, gpu, dt, case):
    Ci, H, W, Co, Hk, Wk, pad, stride, ns = case
    gpu.ptl_set_gemm_path(2)
    try:
        conv_parity(pkg, orc, gpu, dt, Ci, H, W, Co, Hk, Wk, pad, stride, 0, ns, 0xC0DE0051, via_batched=True)
        nd = hp.np_dtype(dt)
        Ho, Wo = hp.conv_out(H, Hk, pad[2], pad[3], stride[0]), hp.conv_out(W, Wk, pad[0], pad[1], stride[1])
        x, dw = dev(np.zeros((ns, Ci, H, W), nd)), dev(np.zeros((Co, Ci, Hk, Wk), nd))
        dy = dev(np.zeros((ns, Co, Ho, Wo), nd))
        a, keep = hp.conv2d_args(pkg, x, None, None, dw, None, dy, Ci, H, W, Co, Hk, Wk, Ho, Wo, pad, stride)
        pkg.call("ptl_conv2d_%s_wg_batched" % dt, a, ns)
        assert gpu.ptl_last_conv_direct() == 1
    finally:
        gpu.ptl_set_gemm_path(0)


# fp16 3x3 layers with one column of padding also take it when rows are whole dwords but not whole 16-byte
# chunks (28, 14, 12, 6 columns): the tile pads every output row to whole chunks.
RAGGED_WG_CASES = [
    # Ci, H, W, Co, ns
    (20, 14, 14, 40, 5),     # two tiles per sample, the second short
    (33, 9, 28, 70, 3),      # two channel slabs, two row tiles
    (8, 6, 6, 9, 7),         # a tile is a whole sample
    (16, 10, 12, 16, 3),
    (4, 5, 26, 6, 2),
]


@pytest.mark.parametrize("case", RAGGED_WG_CASES)
def test_conv2d_direct_weight_gradient_ragged_rows(pkg, orc, gpu, case):
    Ci, H, W, Co, ns = case
    gpu.ptl_set_gemm_path(2)
    try:
        conv_parity(pkg, orc, gpu, "fp16", Ci, H, W, Co, 3, 3, (1, 1, 1, 1), (1, 1), 0, ns, 0xC0DE0052,
                    via_batched=True)
        nd = np.float16
        x, dw = dev(np.zeros((ns, Ci, H, W), nd)), dev(np.zeros((Co, Ci, 3, 3), nd))
        dy = dev(np.zeros((ns, Co, H, W), nd))
        a, keep = hp.conv2d_args(pkg, x, None, None, dw, None, dy, Ci, H, W, Co, 3, 3, H, W, (1, 1, 1, 1), (1, 1))
        pkg.call("ptl_conv2d_fp16_wg_batched", a, ns)
        assert gpu.ptl_last_conv_direct() == 1
    finally:
        gpu.ptl_set_gemm_path(0)


# Wide layers at their real image sizes (too large for the CPU oracle in seconds): forward, weight gradient and
# input gradient against torch's fp32 convolution of the same fp16-rounded tensors, evaluated on the GPU.  The
# checker is torch; the routes these sizes take are the tap-sum product and the resident-tile weight gradient, with 56-wide
# rows (28 row tiles per sample), 28- and 14-wide rows (rows padded to whole chunks inside the tile) and several
# channel slabs.  fp16 outputs are fp32 sums rounded once: 2e-3 relative L2 leaves a factor of five.
@pytest.mark.parametrize("case", [(64, 64, 56, 16), (32, 64, 56, 16), (128, 128, 28, 16), (256, 256, 14, 16),
                                  (128, 128, 16, 32), (64, 64, 8, 128), (128, 256, 14, 32), (512, 512, 7, 32)])
def test_conv2d_wide_layers_against_torch(pkg, gpu, case):
    Ci, Co, H, ns = case
    x = dev(hp.uniform(21, (ns, Ci, H, H), dtype=np.float16))
    w = dev(hp.uniform(22, (Co, Ci, 3, 3), -0.1, 0.1).astype(np.float16))
    dy = dev(hp.uniform(23, (ns, Co, H, H), dtype=np.float16))
    y, dx, dw = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
    a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1), (1, 1))
    for s in ("fw", "wg", "ig"):
        pkg.call("ptl_conv2d_fp16_%s_batched" % s, a, ns)
    sync(gpu)
    xf, wf, dyf = x.float(), w.float(), dy.float()
    ref_y = torch.nn.functional.conv2d(xf, wf, padding=1)
    ref_dw = torch.nn.grad.conv2d_weight(xf, wf.shape, dyf, padding=1)
    ref_dx = torch.nn.grad.conv2d_input(xf.shape, wf, dyf, padding=1)
    for name, got, ref in (("y", y, ref_y), ("dw", dw, ref_dw), ("dx", dx, ref_dx)):
        err = ((got.float() - ref).norm() / ref.norm()).item()
        assert err <= 2e-3, (name, err)


@pytest.mark.parametrize("case", [(256, 256, 32, 32, 16), (128, 256, 20, 45, 24), (256, 128, 30, 30, 40)])
def test_conv2d_resident_tile_weight_gradient_walks_many_units(pkg, gpu, case):
    """The resident-tile weight gradient with eight and more units of 128 positions per workgroup, so that the ring of
    input-tile pieces in LDS goes round several times: rows 33 and 46 wide (the taps reach four 64-position pieces,
    both repeated slots of the ring are read) and 31 wide (three pieces, the widest such row), against torch's fp32
    weight gradient of the same tensors."""
    Ci, Co, H, W, ns = case
    x = dev(hp.uniform(51, (ns, Ci, H, W), dtype=np.float16))
    dy = dev(hp.uniform(53, (ns, Co, H, W), dtype=np.float16))
    w = torch.zeros(Co, Ci, 3, 3, device="cuda").half()
    dw = torch.full_like(w, 3.0)
    a, keep = hp.conv2d_args(pkg, x, None, w, dw, None, dy, Ci, H, W, Co, 3, 3, H, W, (1, 1, 1, 1), (1, 1))
    gpu.ptl_set_gemm_path(5)
    try:
        pkg.call("ptl_conv2d_fp16_wg_batched", a, ns)
        assert gpu.ptl_last_conv_resident() == 1
    finally:
        gpu.ptl_set_gemm_path(0)
    sync(gpu)
    ref = torch.nn.grad.conv2d_weight(x.float(), w.shape, dy.float(), padding=1)
    assert float((dw.float() - ref).norm() / ref.norm()) <= 2e-3
    assert float((dw.float() - ref).abs().max() / ref.abs().max()) <= 5e-3


@pytest.mark.parametrize("case", [(128, 128, 56, 8), (128, 256, 40, 8), (64, 128, 56, 64)])
def test_conv2d_wide_rows_take_the_resident_tile_gradients_by_default(pkg, gpu, case):
    """Rows 41 and 57 wide, filters a multiple of 128: the weight gradient and the one-call backward choose the
    resident-tile kernels by themselves (64 input channels only from 1600 units of positions on); both against
    torch's fp32 gradients of the same tensors, and the one-call backward bit for bit against the two steps."""
    Ci, Co, H, ns = case
    x = dev(hp.uniform(61, (ns, Ci, H, H), dtype=np.float16))
    w = dev(hp.uniform(62, (Co, Ci, 3, 3), -0.1, 0.1).astype(np.float16))
    dy = dev(hp.uniform(63, (ns, Co, H, H), dtype=np.float16))
    dw, dx = torch.full_like(w, 3.0), torch.full_like(x, 3.0)
    a, keep = hp.conv2d_args(pkg, x, dx, w, dw, None, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1), (1, 1))
    pkg.call("ptl_conv2d_fp16_wg_batched", a, ns)
    assert gpu.ptl_last_conv_resident() == 1
    pkg.call("ptl_conv2d_fp16_ig_batched", a, ns)
    sync(gpu)
    ref_dw = torch.nn.grad.conv2d_weight(x.float(), w.shape, dy.float(), padding=1)
    ref_dx = torch.nn.grad.conv2d_input(x.shape, w.float(), dy.float(), padding=1)
    assert float((dw.float() - ref_dw).norm() / ref_dw.norm()) <= 2e-3
    assert float((dx.float() - ref_dx).norm() / ref_dx.norm()) <= 2e-3
    dw2, dx2 = torch.full_like(w, 5.0), torch.full_like(x, 5.0)
    b, keep2 = hp.conv2d_args(pkg, x, dx2, w, dw2, None, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1), (1, 1))
    pkg.call("ptl_conv2d_fp16_bw_batched", b, ns)
    assert gpu.ptl_last_conv_resident() == 1
    sync(gpu)
    assert torch.equal(dw2, dw) and torch.equal(dx2, dx)


def test_conv2d_weight_gradient_of_512_filters_adds_its_partial_sums_the_same_both_ways(pkg, gpu):
    """512 -> 512 on 14x14: the resident-tile weight gradient; its partial sums are added by the kernel that writes the
    nine taps of an output together when dW is 16-byte aligned, by the one that writes them tap by tap when it is
    not - same sums, same bits - and both against torch's fp32 weight gradient."""
    Ci = Co = 512
    H, ns = 14, 16
    x = dev(hp.uniform(31, (ns, Ci, H, H), dtype=np.float16))
    dy = dev(hp.uniform(33, (ns, Co, H, H), dtype=np.float16))
    w = torch.zeros(Co, Ci, 3, 3, device="cuda").half()
    flat = torch.zeros(Co * Ci * 9 + 8, device="cuda").half()
    got = []
    for off in (0, 1):  # (a torch allocation is 256-byte aligned; one element on it is 2-byte aligned)
        dw = flat[off:off + Co * Ci * 9].view(Co, Ci, 3, 3)
        assert dw.data_ptr() % 16 == (0 if off == 0 else 2)
        dw.fill_(3.0)
        a, keep = hp.conv2d_args(pkg, x, None, w, dw, None, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1), (1, 1))
        pkg.call("ptl_conv2d_fp16_wg_batched", a, ns)
        assert gpu.ptl_last_conv_resident() == 1
        sync(gpu)
        got.append(dw.clone())
    assert torch.equal(got[0], got[1])
    ref = torch.nn.grad.conv2d_weight(x.float(), w.shape, dy.float(), padding=1)
    assert float((got[0].float() - ref).norm() / ref.norm()) <= 2e-3


@pytest.mark.parametrize("case", [(64, 64, 56, 8), (128, 128, 28, 16), (256, 256, 14, 32), (64, 128, 12, 64),
                                  (128, 64, 9, 128)])
def test_conv2d_wide_layers_hwc_against_torch(pkg, gpu, case):
    """Channel-minor (HWC) wide 3x3 layers, fp16: forward, weight gradient and input gradient on the sum over taps
    of the padded input, against torch's fp32 convolution of the same tensors."""
    Ci, Co, H, ns = case
    x = dev(hp.uniform(41, (ns, H, H, Ci), dtype=np.float16))
    w = dev(hp.uniform(42, (Co, 3, 3, Ci), -0.1, 0.1).astype(np.float16))
    dy = dev(hp.uniform(43, (ns, H, H, Co), dtype=np.float16))
    y, dx, dw = torch.full_like(dy, 3.0), torch.full_like(x, 3.0), torch.full_like(w, 3.0)
    a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1), (1, 1), 1)
    gpu.ptl_set_gemm_path(3)  # (small batches of narrow layers would otherwise take the gathering GEMM)
    try:
        for s in ("fw", "wg", "ig"):
            pkg.call("ptl_conv2d_fp16_%s_batched" % s, a, ns)
            assert gpu.ptl_last_conv_direct() == 1
    finally:
        gpu.ptl_set_gemm_path(0)
    sync(gpu)
    xf, wf, dyf = (t.float().permute(0, 3, 1, 2).contiguous() for t in (x, w, dy))
    ref_y = torch.nn.functional.conv2d(xf, wf, padding=1).permute(0, 2, 3, 1)
    ref_dw = torch.nn.grad.conv2d_weight(xf, wf.shape, dyf, padding=1).permute(0, 2, 3, 1)
    ref_dx = torch.nn.grad.conv2d_input(xf.shape, wf, dyf, padding=1).permute(0, 2, 3, 1)
    for name, got, ref in (("y", y, ref_y), ("dw", dw, ref_dw), ("dx", dx, ref_dx)):
        err = ((got.float() - ref).norm() / ref.norm()).item()
        assert err <= 2e-3, (name, err)


@pytest.mark.parametrize("case", [(256, 256, 14, 24), (128, 128, 28, 8), (256, 128, 9, 40)])
def test_conv2d_wide_weight_gradient_routes_against_torch(pkg, gpu, case):
    """The weight gradient of a wide layer on each of its routes (default choice, resident-tile kernel, sum over
    taps with its k splits) against torch's fp32 weight gradient of the same fp16-rounded tensors."""
    Ci, Co, H, ns = case
    x = dev(hp.uniform(31, (ns, Ci, H, H), dtype=np.float16))
    dy = dev(hp.uniform(33, (ns, Co, H, H), dtype=np.float16))
    w = torch.zeros(Co, Ci, 3, 3, device=x.device, dtype=torch.float16)
    y, dx = torch.zeros_like(dy), torch.zeros_like(x)
    ref = torch.nn.grad.conv2d_weight(x.float(), w.shape, dy.float(), padding=1)
    try:
        for path in (0, 2, 3):
            gpu.ptl_set_gemm_path(path)
            dw = torch.full_like(w, 7.0)
            a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1), (1, 1))
            pkg.call("ptl_conv2d_fp16_wg_batched", a, ns)
            sync(gpu)
            err = ((dw.float() - ref).norm() / ref.norm()).item()
            assert err <= 2e-3, (path, err)
    finally:
        gpu.ptl_set_gemm_path(0)


def test_conv2d_direct_and_gemm_routes_agree(pkg, gpu):
    """Same forward / input gradient through the direct kernel and through the GEMM route."""
    for dt, tol in (("fp32", 1e-5), ("fp16", 2e-3)):
        nd = hp.np_dtype(dt)
        ns, Ci, Co, H = 160, 16, 32, 32
        x = dev(hp.uniform(7, (ns, Ci, H, H), dtype=nd))
        w = dev(hp.uniform(8, (Co, Ci, 3, 3), dtype=nd))
        dy = dev(hp.uniform(9, (ns, Co, H, H), dtype=nd))
        res = []
        for path in (0, 1):
            gpu.ptl_set_gemm_path(path)
            y, dx, dw = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
            a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1))
            pkg.call("ptl_conv2d_%s_fw_batched" % dt, a, ns)
            assert gpu.ptl_last_conv_direct() == (1 if path == 0 else 0)
            pkg.call("ptl_conv2d_%s_ig_batched" % dt, a, ns)
            assert gpu.ptl_last_conv_direct() == (1 if path == 0 else 0)
            pkg.call("ptl_conv2d_%s_wg_batched" % dt, a, ns)
            assert gpu.ptl_last_conv_direct() == (1 if path == 0 else 0)
            sync(gpu)
            res.append((host(y), host(dx), host(dw)))
        gpu.ptl_set_gemm_path(0)
        for got, ref in zip(res[0], res[1]):
            assert rel_l2(got, ref) <= tol


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
def test_conv2d_naive_selector_and_bias(pkg, orc, gpu, dt):
    conv_parity(pkg, orc, gpu, dt, 4, 10, 10, 6, 3, 3, (1, 1, 1, 1), (1, 1), 0, 1, 0xC0DE0021, im2col=0)
    conv_parity(pkg, orc, gpu, dt, 4, 10, 10, 6, 3, 3, (1, 1, 1, 1), (1, 1), 0, 2, 0xC0DE0022, bias=True)


def test_conv2d_host_pointers_are_staged(pkg, orc, gpu):
    conv_parity(pkg, orc, gpu, "fp32", 4, 10, 10, 6, 3, 3, (1, 1, 1, 1), (1, 1), 0, 1, 0xC0DE0031, host_ptrs=True)
    conv_parity(pkg, orc, gpu, "fp16", 4, 10, 10, 6, 3, 3, (0, 0, 0, 0), (1, 1), 1, 2, 0xC0DE0032, host_ptrs=True)


def test_conv2d_skip_flags(pkg, gpu):
    x = dev(hp.uniform(1, (3, 6, 6)))
    w = dev(hp.uniform(2, (4, 3, 3, 3)))
    dy = dev(hp.uniform(3, (4, 4, 4)))
    dx, dw = dev(np.full((3, 6, 6), 9, np.float32)), dev(np.full((4, 3, 3, 3), 9, np.float32))
    g, keep = hp.conv2d_args(pkg, x, dx, w, dw, None, dy, 3, 6, 6, 4, 3, 3, 4, 4)
    g.skip_wg_grad, g.skip_in_grad = 1, 0
    pkg.call("pulp_conv2d_fp32_bw_cl", g)
    sync(gpu)
    assert torch.all(dw == 9) and not torch.any(dx == 9)


# --------------------------------------------------------------------------- pointwise
def pw_parity(pkg, orc, lib, dt, Ci, Co, H, W, hwc, ns, seed):
    nd = hp.np_dtype(dt)
    xs = (ns, H * W, Ci) if hwc else (ns, Ci, H * W)
    ys = (ns, H * W, Co) if hwc else (ns, Co, H * W)
    ws = (Ci, Co) if (hwc and dt == "fp32") else (Co, Ci)
    x, w, dy = hp.uniform(seed, xs, dtype=nd), hp.uniform(seed + 1, ws, dtype=nd), hp.uniform(seed + 2, ys, dtype=nd)
    y, dx, dw = np.zeros(ys, nd), np.zeros(xs, nd), np.zeros(ws, nd)
    a, keep = hp.pw_args(pkg, x, dx, w, dw, y, dy, Ci, Co, H, W, hwc)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_conv_pw_" + s, dt, a, ns)
    gx, gw, gdy = dev(x), dev(w), dev(dy)
    gy, gdx, gdw = dev(np.full(ys, 3, nd)), dev(np.full(xs, 3, nd)), dev(np.full(ws, 3, nd))
    g, keep2 = hp.pw_args(pkg, gx, gdx, gw, gdw, gy, gdy, Ci, Co, H, W, hwc)
    if ns == 1:
        pkg.call("pulp_conv_pw_%s_fw_cl" % dt, g)
        pkg.call("pulp_conv_pw_%s_bw_cl" % dt, g)
    else:
        for s in ("fw", "wg", "ig"):
            pkg.call("ptl_conv_pw_%s_%s_batched" % (dt, s), g, ns)
    sync(lib)
    errs = {}
    for name, got, ref in (("y", gy, y), ("dw", gdw, dw), ("dx", gdx, dx)):
        errs[name] = rel_l2(host(got), ref)
        assert errs[name] <= TOL[dt], (name, errs[name])
    return errs


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("Ci,Co,H,W,ns", [(8, 8, 8, 8, 1), (8, 16, 7, 9, 1), (64, 128, 56, 56, 1), (24, 40, 10, 10, 4)])
def test_pointwise(pkg, orc, gpu, dt, hwc, Ci, Co, H, W, ns):
    pw_parity(pkg, orc, gpu, dt, Ci, Co, H, W, hwc, ns, 0xC0DE0003)


# Batches large enough for the streaming kernel (row panel resident, column tiles streamed): one or two row
# tiles, contraction depths of one, two and four slabs over the two data types and the two steps.
@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("Ci,Co,H,W,ns", [(64, 128, 32, 32, 64), (128, 64, 32, 32, 64), (64, 256, 16, 16, 256)])
def test_pointwise_streamed_column_tiles(pkg, orc, gpu, dt, hwc, Ci, Co, H, W, ns):
    """Channel-major layers stream pixel columns past a resident weight panel; pixel-major (HWC) layers are the
    same product transposed, stored four channels at a time."""
    pw_parity(pkg, orc, gpu, dt, Ci, Co, H, W, hwc, ns, 0xC0DE0043)
    nd = hp.np_dtype(dt)
    x = dev(hp.uniform(1, (ns, H * W, Ci) if hwc else (ns, Ci, H * W), dtype=nd))
    w = dev(hp.uniform(2, (Ci, Co) if (hwc and dt == "fp32") else (Co, Ci), dtype=nd))
    y = torch.zeros((ns, H * W, Co) if hwc else (ns, Co, H * W), dtype=x.dtype, device=x.device)
    g, keep = hp.pw_args(pkg, x, None, w, None, y, None, Ci, Co, H, W, hwc)
    pkg.call("ptl_conv_pw_%s_fw_batched" % dt, g, ns)
    sync(gpu)
    assert gpu.ptl_last_gemm_streamed() == 1
    wm = w.double().t() if (hwc and dt == "fp32") else w.double()  # [Co][Ci]
    ref = torch.matmul(x.double(), wm.t()) if hwc else torch.matmul(wm, x.double())
    assert float((y.double() - ref).norm() / ref.norm()) <= TOL[dt]


# --------------------------------------------------------------------------- depthwise
def dw_parity(pkg, orc, lib, dt, C, H, W, K, pad, stride, ns, seed):
    L, R, U, D = pad
    Ho, Wo = hp.conv_out(H, K, U, D, stride[0]), hp.conv_out(W, K, L, R, stride[1])
    nd = hp.np_dtype(dt)
    x = hp.uniform(seed, (ns, C, H, W), dtype=nd)
    w = hp.uniform(seed + 1, (C, K, K), dtype=nd)
    dy = hp.uniform(seed + 2, (ns, C, Ho, Wo), dtype=nd)
    y, dx, dw = np.zeros_like(dy), np.zeros_like(x), np.zeros_like(w)
    a, keep = hp.dw_args(pkg, dt, x, dx, w, dw, y, dy, C, H, W, K, K, Ho, Wo, pad, stride)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_conv_dw_" + s, dt, a, ns)
    gx, gw, gdy = dev(x), dev(w), dev(dy)
    gy, gdx, gdw = dev(np.full(dy.shape, 3, nd)), dev(np.full(x.shape, 3, nd)), dev(np.full(w.shape, 3, nd))
    g, keep2 = hp.dw_args(pkg, dt, gx, gdx, gw, gdw, gy, gdy, C, H, W, K, K, Ho, Wo, pad, stride)
    if ns == 1:
        pkg.call("pulp_conv_dw_%s_fw_cl" % dt, g)
        pkg.call("pulp_conv_dw_%s_bw_cl" % dt, g)
    else:
        for s in ("fw", "wg", "ig"):
            pkg.call("ptl_conv_dw_%s_%s_batched" % (dt, s), g, ns)
    sync(lib)
    for name, got, ref in (("y", gy, y), ("dw", gdw, dw), ("dx", gdx, dx)):
        e = rel_l2(host(got), ref)
        assert e <= TOL[dt], (name, e)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("C,H,W,K,pad,ns", [(8, 9, 9, 3, (0, 0, 0, 0), 1), (64, 58, 58, 3, (0, 0, 0, 0), 1),
                                            (16, 12, 10, 5, (0, 0, 0, 0), 3), (8, 9, 9, 3, (1, 1, 1, 1), 2)])
def test_depthwise(pkg, orc, gpu, dt, C, H, W, K, pad, ns):
    dw_parity(pkg, orc, gpu, dt, C, H, W, K, pad, (1, 1), ns, 0xC0DE0103)


# Batches with at least two planes per CU run the plane-resident kernels: even and odd row lengths (fp16 rows of
# even length are read as pairs of neighbours), 3x3 and 5x5, and padded fp32 planes.
# fp16 3x3 planes whose output rows are whole 16-byte groups load their blocks straight from global memory (forward;
# the weight gradient whenever rows are whole dwords): full and ragged row blocks, an even left pad.
@pytest.mark.parametrize("dt,C,H,W,K,pad,ns", [("fp16", 64, 34, 34, 3, (0, 0, 0, 0), 8), ("fp16", 64, 23, 32, 3, (2, 0, 1, 1), 8),
                                               ("fp16", 64, 36, 36, 3, (0, 0, 0, 0), 8), ("fp16", 64, 35, 37, 3, (0, 0, 0, 0), 8),
                                               ("fp16", 32, 38, 40, 5, (0, 0, 0, 0), 16), ("fp16", 32, 37, 39, 5, (0, 0, 0, 0), 16),
                                               ("fp32", 64, 36, 36, 3, (0, 0, 0, 0), 8), ("fp32", 64, 35, 37, 3, (1, 1, 1, 1), 8),
                                               ("fp32", 32, 38, 38, 5, (2, 2, 2, 2), 16)])
def test_depthwise_plane_resident(pkg, orc, gpu, dt, C, H, W, K, pad, ns):
    dw_parity(pkg, orc, gpu, dt, C, H, W, K, pad, (1, 1), ns, 0xC0DE0105)


def test_depthwise_fp32_stride_and_padding(pkg, orc, gpu):
    dw_parity(pkg, orc, gpu, "fp32", 6, 11, 11, 3, (1, 1, 1, 1), (2, 2), 2, 0xC0DE0104)


# ------------------------------------------------------------------------------ Linear
def linear_parity(pkg, orc, lib, dt, n_in, n_out, ns, seed, bias=False):
    nd = hp.np_dtype(dt)
    x = hp.normal(seed, (ns, n_in), 1.0 / np.sqrt(n_in), nd)
    w = hp.normal(seed + 1, (n_out, n_in), 1.0 / np.sqrt(n_in), nd)
    dy = hp.uniform(seed + 2, (ns, n_out), dtype=nd)
    b = hp.uniform(seed + 3, (n_out,), dtype=nd) if bias else None
    y, dx, dw = np.zeros_like(dy), np.zeros_like(x), np.zeros_like(w)
    db = np.zeros((n_out,), nd) if bias else None
    a, keep = hp.linear_args(pkg, x, dx, w, dw, y, dy, n_in, n_out, b, db)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_linear_" + s, dt, a, ns)
    gx, gw, gdy, gb = dev(x), dev(w), dev(dy), dev(b)
    gy, gdx, gdw = dev(np.full(dy.shape, 3, nd)), dev(np.full(x.shape, 3, nd)), dev(np.full(w.shape, 3, nd))
    gdb = dev(np.full((n_out,), 3, nd)) if bias else None
    g, keep2 = hp.linear_args(pkg, gx, gdx, gw, gdw, gy, gdy, n_in, n_out, gb, gdb)
    if ns == 1:
        pkg.call("pulp_linear_%s_fw_cl" % dt, g)
        pkg.call("pulp_linear_%s_bw_cl" % dt, g)
    else:
        for s in ("fw", "wg", "ig"):
            pkg.call("ptl_linear_%s_%s_batched" % (dt, s), g, ns)
    sync(lib)
    out = [("y", gy, y), ("dw", gdw, dw), ("dx", gdx, dx)]
    if bias:
        out.append(("db", gdb, db))
    errs = {}
    for name, got, ref in out:
        errs[name] = rel_l2(host(got), ref)
        assert errs[name] <= TOL[dt], (name, errs[name])
    return errs


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("n_in,n_out,ns", [(8, 8, 1), (1024, 8, 1), (1024, 1024, 1), (100, 37, 1), (1024, 1024, 512),
                                           (72, 50, 9)])
def test_linear(pkg, orc, gpu, dt, n_in, n_out, ns):
    linear_parity(pkg, orc, gpu, dt, n_in, n_out, ns, 0xC0DE0002)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
def test_linear_bias(pkg, orc, gpu, dt):
    linear_parity(pkg, orc, gpu, dt, 64, 48, 1, 0xC0DE0202, bias=True)
    linear_parity(pkg, orc, gpu, dt, 64, 48, 6, 0xC0DE0203, bias=True)


# ---------------------------------------------------------------------- mm / mm_manager
@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("n_in,n_out,ns", [(1024, 1024, 512), (1024, 1024, 384), (1024, 896, 320), (256, 384, 640), (100, 37, 9), (64, 64, 1)])
def test_linear_bw_batched_matches_separate_steps(pkg, gpu, dt, n_in, n_out, ns):
    """ptl_linear_*_bw_batched (weight + input gradient in one call) against the two single steps."""
    nd = hp.np_dtype(dt)
    x = dev(hp.normal(11, (ns, n_in), 1.0 / 16.0, nd))
    w = dev(hp.normal(12, (n_out, n_in), 1.0 / 16.0, nd))
    dy = dev(hp.uniform(13, (ns, n_out), dtype=nd))
    res = []
    for both in (False, True):
        y = torch.zeros(ns, n_out, dtype=x.dtype, device=DEV)
        dx, dw = torch.full_like(x, 3), torch.full_like(w, 3)
        a, keep = hp.linear_args(pkg, x, dx, w, dw, y, dy, n_in, n_out)
        if both:
            pkg.call("ptl_linear_%s_bw_batched" % dt, a, ns)
        else:
            pkg.call("ptl_linear_%s_wg_batched" % dt, a, ns)
            pkg.call("ptl_linear_%s_ig_batched" % dt, a, ns)
        sync(gpu)
        res.append((host(dw), host(dx)))
    tol = 1e-6 if dt == "fp32" else 2e-3
    assert rel_l2(res[1][0], res[0][0]) <= tol
    assert rel_l2(res[1][1], res[0][1]) <= tol
    # skip flags select one of the two
    dx, dw = torch.full_like(x, 3), torch.full_like(w, 3)
    y = torch.zeros(ns, n_out, dtype=x.dtype, device=DEV)
    a, keep = hp.linear_args(pkg, x, dx, w, dw, y, dy, n_in, n_out)
    a.skip_in_grad = 1
    pkg.call("ptl_linear_%s_bw_batched" % dt, a, ns)
    sync(gpu)
    assert rel_l2(host(dw), res[0][0]) <= tol
    assert np.all(host(dx) == 3)


@pytest.mark.parametrize("dt", ["fp32", "fp16"])
@pytest.mark.parametrize("N,M,K", [(32, 32, 32), (32, 1024, 144), (32, 144, 1024), (16, 1024, 288), (128, 3136, 64),
                                   (7, 5, 3), (1, 33, 20), (33, 1, 20), (9, 11, 1), (130, 70, 515)])
def test_mm_family(pkg, orc, gpu, dt, N, M, K):
    nd = hp.np_dtype(dt)
    for tb in (0, 1):
        A = hp.normal(5, (N, K), 1.0 / np.sqrt(K), nd)
        B = hp.uniform(6, (M, K) if tb else (K, M), dtype=nd)
        C = np.zeros((N, M), nd)
        orc.call("orc_mm", dt, hp.mm_args(pkg, A, B, C, N, M, K, tb))
        gA, gB, gC = dev(A), dev(B), dev(np.full((N, M), 3, nd))
        m = hp.mm_args(pkg, gA, gB, gC, N, M, K, tb)
        name = "mm" if dt == "fp32" else "mm_fp16"
        pkg.call(name, m)
        sync(gpu)
        assert rel_l2(host(gC), C) <= TOL[dt]
        # through the dispatcher, every id of the list gives the same product
        man = pkg.MMManagerArgs()
        man.mm_args = ctypes.pointer(m)
        for mid in ((0, 1, 10, 23) if dt == "fp32" else (0, 3, 8)):
            gC.fill_(3)
            man.layer_type, man.step_type, man.matmul_type = pkg.LAYER_CONV2D, pkg.STEP_FW, mid
            pkg.call("mm_manager" if dt == "fp32" else "mm_manager_fp16", man)
            sync(gpu)
            assert rel_l2(host(gC), C) <= TOL[dt]


@pytest.mark.parametrize("N,M,K", [(4096, 2048, 256), (4000, 2040, 192), (66000, 64, 128), (65536, 48, 192)])
def test_mm_fp16_large_and_tall_tiles(pkg, gpu, N, M, K):
    """fp16 products that give every CU a 256x128 tile, and narrow ones on the 128x64 tile; whole and ragged,
    against torch in float32."""
    g = torch.Generator(device="cpu").manual_seed(17)
    A = (torch.randn(N, K, generator=g) / 8).half().to(DEV)
    for tb in (0, 1):
        B = (torch.randn((M, K) if tb else (K, M), generator=g) / 8).half().to(DEV)
        C = torch.full((N, M), 3, dtype=torch.float16, device=DEV)
        pkg.call("mm_fp16", hp.mm_args(pkg, A, B, C, N, M, K, tb))
        sync(gpu)
        ref = A.float() @ (B.float().t() if tb else B.float())
        assert float((C.float() - ref).norm() / ref.norm()) <= 1e-3
        assert float((C.float() - ref).abs().max()) <= 2e-2


@pytest.mark.parametrize("N,M,K", [(4096, 4096, 512), (4090, 4000, 192)])
def test_mm_fp16_square_tiles_with_chunked_epilogue(pkg, gpu, N, M, K):
    """fp16 products with more than 256 tall tiles take the 256x256 tile, whose accumulators are parked and stored
    in four passes; whole and ragged, both orientations of B, against torch in float32."""
    g = torch.Generator(device="cpu").manual_seed(23)
    A = (torch.randn(N, K, generator=g) / 8).half().to(DEV)
    for tb in (0, 1):
        B = (torch.randn((M, K) if tb else (K, M), generator=g) / 8).half().to(DEV)
        C = torch.full((N, M), 3, dtype=torch.float16, device=DEV)
        pkg.call("mm_fp16", hp.mm_args(pkg, A, B, C, N, M, K, tb))
        sync(gpu)
        assert gpu.ptl_last_gemm_tile() == 256 * 1000 + 256, gpu.ptl_last_gemm_tile()
        ref = A.float() @ (B.float().t() if tb else B.float())
        assert float((C.float() - ref).norm() / ref.norm()) <= 1e-3
        assert float((C.float() - ref).abs().max()) <= 2e-2


def test_mm_k0_leaves_output_untouched(pkg, gpu):
    gA, gB, gC = dev(np.zeros((3, 1), np.float32)), dev(np.zeros((1, 4), np.float32)), dev(np.full((3, 4), 5, np.float32))
    pkg.call("mm", hp.mm_args(pkg, gA, gB, gC, 3, 4, 0, 0))
    sync(gpu)
    assert torch.all(gC == 5)


def test_mm_reference_closed_form(pkg, gpu):
    """A, B of tests/test_matmul (32x32x32, divider 1e8) against numpy float64."""
    N = K = M = 32
    i, j = np.meshgrid(np.arange(N), np.arange(K), indexing="ij")
    A = ((1.0 + (i + j + 0.1)) / 1e8).astype(np.float32)
    B = (i * j + 0.1).astype(np.float32)
    gA, gB, gC = dev(A), dev(B), dev(np.zeros((N, M), np.float32))
    pkg.call("mm", hp.mm_args(pkg, gA, gB, gC, N, M, K, 0))
    sync(gpu)
    assert rel_l2(host(gC), A.astype(np.float64) @ B.astype(np.float64)) < 1e-6


# ---------------------------------------------------------------- fp16: the second distance
# The fp16 oracle accumulates in fp16 as the reference does and is itself 5e-3 away from the exact result, so the
# 1e-2 bar against it cannot see a kernel error of that size.  The library accumulates in fp32 and rounds once:
# against the fp32 oracle fed the same fp16-rounded tensors it must be within 1e-3 (measured 2-4e-4 = the
# rounding of the stored result) on every BASELINE shape the fp16 path serves.
TIGHT = 1e-3


def _tight(got, ref, what):
    e = rel_l2(host(got).astype(np.float32), ref)
    assert e <= TIGHT, (what, e)


@pytest.mark.parametrize("hwc", [0, 1])
@pytest.mark.parametrize("ns", [1, 6])
def test_fp16_conv2d_config1_against_fp32_oracle(pkg, orc, gpu, hwc, ns):
    Ci, H, Co, K = 16, 32, 32, 3
    xs = (ns, H, H, Ci) if hwc else (ns, Ci, H, H)
    ws = (Co, K, K, Ci) if hwc else (Co, Ci, K, K)
    ys = (ns, H, H, Co) if hwc else (ns, Co, H, H)
    x, w, dy = (hp.uniform(0xC0DE0501 + i, s, dtype=np.float16) for i, s in enumerate((xs, ws, ys)))
    xf, wf, dyf = (v.astype(np.float32) for v in (x, w, dy))
    y, dx, dw = np.zeros(ys, np.float32), np.zeros(xs, np.float32), np.zeros(ws, np.float32)
    a, keep = hp.conv2d_args(pkg, xf, dx, wf, dw, y, dyf, Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1), (1, 1), hwc)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_conv2d_" + s, "fp32", a, ns)
    gy, gdx, gdw = (dev(np.full(s, 3, np.float16)) for s in (ys, xs, ws))
    g, keep2 = hp.conv2d_args(pkg, dev(x), gdx, dev(w), gdw, gy, dev(dy), Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1), (1, 1),
                              hwc)
    if ns == 1:
        pkg.call("pulp_conv2d_fp16_fw_cl", g)
        pkg.call("pulp_conv2d_fp16_bw_cl", g)
    else:
        for s in ("fw", "wg", "ig"):
            pkg.call("ptl_conv2d_fp16_%s_batched" % s, g, ns)
    sync(gpu)
    for name, got, ref in (("y", gy, y), ("dw", gdw, dw), ("dx", gdx, dx)):
        _tight(got, ref, name)


@pytest.mark.parametrize("ns", [1, 512])
def test_fp16_linear_config2_against_fp32_oracle(pkg, orc, gpu, ns):
    n = 1024
    x = hp.normal(0xC0DE0511, (ns, n), 1.0 / 32, np.float16)
    w = hp.normal(0xC0DE0512, (n, n), 1.0 / 32, np.float16)
    dy = hp.uniform(0xC0DE0513, (ns, n), dtype=np.float16)
    xf, wf, dyf = (v.astype(np.float32) for v in (x, w, dy))
    y, dx, dw = np.zeros_like(dyf), np.zeros_like(xf), np.zeros_like(wf)
    a, keep = hp.linear_args(pkg, xf, dx, wf, dw, y, dyf, n, n)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_linear_" + s, "fp32", a, ns)
    gy, gdx, gdw = (dev(np.full(v.shape, 3, np.float16)) for v in (dy, x, w))
    g, keep2 = hp.linear_args(pkg, dev(x), gdx, dev(w), gdw, gy, dev(dy), n, n)
    if ns == 1:
        pkg.call("pulp_linear_fp16_fw_cl", g)
        pkg.call("pulp_linear_fp16_bw_cl", g)
    else:
        pkg.call("ptl_linear_fp16_fw_batched", g, ns)
        pkg.call("ptl_linear_fp16_bw_batched", g, ns)
    sync(gpu)
    for name, got, ref in (("y", gy, y), ("dw", gdw, dw), ("dx", gdx, dx)):
        _tight(got, ref, name)


@pytest.mark.parametrize("ns", [1, 8])
def test_fp16_depthwise_pointwise_config3_against_fp32_oracle(pkg, orc, gpu, ns):
    """Depthwise 3x3 on 64 x 56 x 56 (stored pre-padded to 58 x 58, as the fp16 depthwise layer has no padding of
    its own) and pointwise 64 -> 128; the fp32 depthwise oracle takes the same pre-padded tensor."""
    C, Co, Hp, Ho, K = 64, 128, 58, 56, 3
    x = hp.uniform(0xC0DE0521, (ns, C, Hp, Hp), dtype=np.float16)
    w = hp.uniform(0xC0DE0522, (C, K, K), dtype=np.float16)
    dy = hp.uniform(0xC0DE0523, (ns, C, Ho, Ho), dtype=np.float16)
    xf, wf, dyf = (v.astype(np.float32) for v in (x, w, dy))
    y, dx, dw = np.zeros_like(dyf), np.zeros_like(xf), np.zeros_like(wf)
    a, keep = hp.dw_args(pkg, "fp32", xf, dx, wf, dw, y, dyf, C, Hp, Hp, K, K, Ho, Ho)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_conv_dw_" + s, "fp32", a, ns)
    gy, gdx, gdw = (dev(np.full(v.shape, 3, np.float16)) for v in (dy, x, w))
    g, keep2 = hp.dw_args(pkg, "fp16", dev(x), gdx, dev(w), gdw, gy, dev(dy), C, Hp, Hp, K, K, Ho, Ho)
    if ns == 1:
        pkg.call("pulp_conv_dw_fp16_fw_cl", g)
        pkg.call("pulp_conv_dw_fp16_bw_cl", g)
    else:
        for s in ("fw", "wg", "ig"):
            pkg.call("ptl_conv_dw_fp16_%s_batched" % s, g, ns)
    sync(gpu)
    for name, got, ref in (("dw y", gy, y), ("dw dw", gdw, dw), ("dw dx", gdx, dx)):
        _tight(got, ref, name)
    # pointwise on the depthwise output
    px = host(gy)
    pw_ = hp.uniform(0xC0DE0524, (Co, C), dtype=np.float16)
    pdy = hp.uniform(0xC0DE0525, (ns, Co, Ho * Ho), dtype=np.float16)
    pxf, pwf, pdyf = (v.astype(np.float32) for v in (px, pw_, pdy))
    py, pdx, pdw = np.zeros_like(pdyf), np.zeros_like(pxf), np.zeros_like(pwf)
    a, keep = hp.pw_args(pkg, pxf, pdx, pwf, pdw, py, pdyf, C, Co, Ho, Ho)
    for s in ("fw", "wg", "ig"):
        orc.call("orc_conv_pw_" + s, "fp32", a, ns)
    gpy, gpdx, gpdw = (dev(np.full(v.shape, 3, np.float16)) for v in (pdy, px, pw_))
    g, keep2 = hp.pw_args(pkg, gy, gpdx, dev(pw_), gpdw, gpy, dev(pdy), C, Co, Ho, Ho)
    if ns == 1:
        pkg.call("pulp_conv_pw_fp16_fw_cl", g)
        pkg.call("pulp_conv_pw_fp16_bw_cl", g)
    else:
        for s in ("fw", "wg", "ig"):
            pkg.call("ptl_conv_pw_fp16_%s_batched" % s, g, ns)
    sync(gpu)
    for name, got, ref in (("pw y", gpy, py), ("pw dw", gpdw, pdw), ("pw dx", gpdx, pdx)):
        _tight(got, ref, name)
