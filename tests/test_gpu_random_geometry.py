"""Randomised geometries (fixed seeds) through the fp16 convolution and depthwise kernels whose index arithmetic
depends on the image size: the resident-tile Conv2D kernels (forward, input gradient, weight gradient, both
gradients in one call) and the depthwise kernels, against torch in float32.  The oracle checks in
test_gpu_parity.py pin the arithmetic; these cases sweep row lengths, paddings and batch sizes for ragged tiles,
sample boundaries inside a tile, partial column groups and plane edges."""
import ctypes
import random

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import helpers as hp

pytestmark = pytest.mark.gpu


def rel(got, ref):
    return float((got.to(ref.dtype) - ref).norm() / (ref.norm() + 1e-20))


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_conv2d_resident_tile_random_geometries(pkg, gpu, seed):
    rng = random.Random(seed)
    for it in range(14):
        Ci, Co = rng.choice([64, 64, 128, 192]), rng.choice([64, 128, 128, 192, 256])
        pl, pr, pu, pd = (rng.randint(0, 2) for _ in range(4))
        W, H = rng.randint(max(3 - pl - pr, 1), 61 - pl - pr), rng.randint(max(3 - pu - pd, 1), 40)
        ns = rng.choice([1, 2, 3, 5, 8, 17, 40])
        Ho, Wo = H + pu + pd - 2, W + pl + pr - 2
        x = (torch.rand(ns, Ci, H, W, device="cuda") - 0.5).half()
        w = ((torch.rand(Co, Ci, 3, 3, device="cuda") - 0.5) * 0.2).half()
        dy = (torch.rand(ns, Co, Ho, Wo, device="cuda") - 0.5).half()
        y, dx, dw = torch.full_like(dy, 3), torch.full_like(x, 3), torch.full_like(w, 3)
        dx2, dw2 = torch.full_like(x, 3), torch.full_like(w, 3)
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, (pl, pr, pu, pd), (1, 1))
        a2, keep2 = hp.conv2d_args(pkg, x, dx2, w, dw2, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, (pl, pr, pu, pd), (1, 1))
        gpu.ptl_set_gemm_path(5)
        try:
            for s in ("fw", "ig", "wg"):
                pkg.call("ptl_conv2d_fp16_%s_batched" % s, a, ns)
            pkg.call("ptl_conv2d_fp16_bw_batched", a2, ns)
        finally:
            gpu.ptl_set_gemm_path(0)
        gpu.ptl_sync()
        xp = F.pad(x.float(), (pl, pr, pu, pd))
        ref_y = F.conv2d(xp, w.float())
        ref_dx = torch.nn.grad.conv2d_input(xp.shape, w.float(), dy.float())[:, :, pu:pu + H, pl:pl + W]
        ref_dw = torch.nn.grad.conv2d_weight(xp, w.shape, dy.float())
        case = (Ci, Co, H, W, (pl, pr, pu, pd), ns)
        for name, got, ref in (("y", y, ref_y), ("dx", dx, ref_dx), ("dw", dw, ref_dw), ("dx one call", dx2, ref_dx),
                               ("dw one call", dw2, ref_dw)):
            assert rel(got, ref) <= 2e-3, (case, name)


@pytest.mark.parametrize("dt,seed", [("fp16", 31), ("fp16", 32), ("fp16", 33), ("fp32", 34), ("fp32", 35)])
def test_conv2d_small_layer_kernel_random_geometries(pkg, gpu, dt, seed):
    """The single-launch kernels for small 3x3 layers (forced with path 6): channel counts that are not whole
    blocks (3, 24, 40 ...), strides 1 and 2, paddings 0..2 per side, rows of 8..64 elements, ragged last row tiles."""
    rng = random.Random(seed)
    tdt, tol = (torch.float16, 2e-3) if dt == "fp16" else (torch.float32, 2e-5)
    ran = 0
    for it in range(16):
        Ci, Co = rng.choice([3, 8, 16, 24, 32, 48, 64]), rng.choice([8, 16, 24, 32, 40, 64])
        st = rng.choice([1, 1, 2])
        pl, pr, pu, pd = (rng.randint(0, 2) for _ in range(4))
        W, H = rng.choice([8, 16, 24, 32, 40, 64] if dt == "fp16" else [8, 12, 16, 20, 32, 40]), rng.randint(3, 36)
        if st == 2:  # the strides must divide the padded extents minus the filter
            pr += (W + pl + pr - 3) % 2
            pd += (H + pu + pd - 3) % 2
        ns = rng.choice([1, 2, 3, 7, 32, 130])
        Ho, Wo = (H + pu + pd - 3) // st + 1, (W + pl + pr - 3) // st + 1
        x = (torch.rand(ns, Ci, H, W, device="cuda") - 0.5).to(tdt)
        w = ((torch.rand(Co, Ci, 3, 3, device="cuda") - 0.5) * 0.5).to(tdt)
        dy = (torch.rand(ns, Co, Ho, Wo, device="cuda") - 0.5).to(tdt)
        y, dx, dw = torch.full_like(dy, 3), torch.full_like(x, 3), torch.full_like(w, 3)
        dx2, dw2 = torch.full_like(x, 3), torch.full_like(w, 3)
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, (pl, pr, pu, pd), (st, st))
        a2, keep2 = hp.conv2d_args(pkg, x, dx2, w, dw2, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, (pl, pr, pu, pd), (st, st))
        case = (Ci, Co, H, W, (pl, pr, pu, pd), st, ns)
        gpu.ptl_set_gemm_path(6)
        try:
            pkg.call("ptl_conv2d_%s_fw_batched" % dt, a, ns)
            small_fw = gpu.ptl_last_conv_resident() == 2
            pkg.call("ptl_conv2d_%s_ig_batched" % dt, a, ns)
            small_ig = gpu.ptl_last_conv_resident() == 2
            # the weight gradient (alone, and with the input gradient in the same launch): whatever route takes it
            pkg.call("ptl_conv2d_%s_wg_batched" % dt, a, ns)
            pkg.call("ptl_conv2d_%s_bw_batched" % dt, a2, ns)
        finally:
            gpu.ptl_set_gemm_path(0)
        gpu.ptl_sync()
        # the kernel fits when the filter tensor is whole 16-byte pieces and one row of every channel block is at most
        # 64 wave-wide loads; the input gradient sees the output gradient as its input (zero-stuffed in the kernel for a
        # stride-2 layer), whose rows must be whole pieces too
        blocks = lambda c: (16 if c <= 16 else 32 if c <= 32 else 64) // 8
        if dt == "fp16":
            assert small_fw == ((Ci * Co * 9) % 8 == 0 and blocks(Ci) * (W // 8) <= 64), case
            assert small_ig == (Wo % 8 == 0 and (Ci * Co * 9) % 8 == 0 and blocks(Co) * (Wo // 8) <= 64), case
        ran += small_fw + small_ig
        xp = F.pad(x.double(), (pl, pr, pu, pd))
        ref_y = F.conv2d(xp, w.double(), stride=st)
        ref_dx = torch.nn.grad.conv2d_input(xp.shape, w.double(), dy.double(), stride=st)[:, :, pu:pu + H, pl:pl + W]
        ref_dw = torch.nn.grad.conv2d_weight(xp, w.shape, dy.double(), stride=st)
        assert rel(y, ref_y) <= tol, (case, "y")
        assert rel(dx, ref_dx) <= tol, (case, "dx")
        assert rel(dw, ref_dw) <= tol, (case, "dw")
        assert rel(dx2, ref_dx) <= tol, (case, "dx, one call")
        assert rel(dw2, ref_dw) <= tol, (case, "dw, one call")
    assert ran >= (12 if dt == "fp16" else 8)


@pytest.mark.parametrize("dt,seed", [("fp16", 41), ("fp16", 42), ("fp32", 43), ("fp32", 44)])
def test_conv2d_small_layer_weight_gradient_random_geometries(pkg, gpu, dt, seed):
    """Unit-stride 3x3 fp16 layers whose output is as wide as the input (the geometries the small-layer weight-gradient
    kernel takes, forced with path 6): weight gradient alone and together with the input gradient, tiles of several
    samples (64 channels), split rows (few samples), ragged last tiles, all three left paddings."""
    rng = random.Random(seed)
    tdt, tol, vec = (torch.float16, 2e-3, 8) if dt == "fp16" else (torch.float32, 2e-5, 4)
    for it in range(14):
        Ci, Co = rng.choice([3, 8, 16, 24, 32, 64]), rng.choice([8, 16, 32, 40, 64])
        pl = rng.randint(0, 2)
        pr, pu, pd = 2 - pl, rng.randint(0, 2), rng.randint(0, 2)
        W, H = rng.choice([8, 16, 24, 32] if dt == "fp16" else [8, 12, 16, 20, 32]), rng.randint(max(3 - pu - pd, 1), 34)
        ns = rng.choice([1, 2, 5, 9, 32, 130])
        Ho, Wo = H + pu + pd - 2, W
        x = (torch.rand(ns, Ci, H, W, device="cuda") - 0.5).to(tdt)
        w = ((torch.rand(Co, Ci, 3, 3, device="cuda") - 0.5) * 0.5).to(tdt)
        dy = (torch.rand(ns, Co, Ho, Wo, device="cuda") - 0.5).to(tdt)
        y, dx, dw = torch.full_like(dy, 3), torch.full_like(x, 3), torch.full_like(w, 3)
        dx2, dw2 = torch.full_like(x, 3), torch.full_like(w, 3)
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, (pl, pr, pu, pd), (1, 1))
        a2, keep2 = hp.conv2d_args(pkg, x, dx2, w, dw2, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, (pl, pr, pu, pd), (1, 1))
        case = (Ci, Co, H, W, (pl, pr, pu, pd), ns)
        gpu.ptl_set_gemm_path(6)
        try:
            pkg.call("ptl_conv2d_%s_wg_batched" % dt, a, ns)
            pkg.call("ptl_conv2d_%s_bw_batched" % dt, a2, ns)
            if dt == "fp16":
                assert gpu.ptl_last_conv_resident() == (2 if (Ci * Co * 9) % 8 == 0 else 0), case
        finally:
            gpu.ptl_set_gemm_path(0)
        gpu.ptl_sync()
        xp = F.pad(x.double(), (pl, pr, pu, pd))
        ref_dx = torch.nn.grad.conv2d_input(xp.shape, w.double(), dy.double())[:, :, pu:pu + H, pl:pl + W]
        ref_dw = torch.nn.grad.conv2d_weight(xp, w.shape, dy.double())
        assert rel(dw, ref_dw) <= tol, (case, "dw")
        assert rel(dx2, ref_dx) <= tol, (case, "dx, one call")
        assert rel(dw2, ref_dw) <= tol, (case, "dw, one call")


@pytest.mark.parametrize("dt,seed", [("fp16", 51), ("fp16", 52), ("fp32", 53)])
def test_conv2d_small_layer_stride2_gradients_random_geometries(pkg, gpu, dt, seed):
    """3x3 layers at stride 2 with one column of left padding and an even input width (what the small-layer
    weight-gradient kernel takes at that stride, forced with path 6): weight gradient alone and both gradients in
    one call, against torch in float64; the ResNet-20 shapes among them."""
    rng = random.Random(seed)
    tdt, tol, vec = (torch.float16, 2e-3, 8) if dt == "fp16" else (torch.float32, 2e-5, 4)
    fixed = [(16, 32, 32, 32, 1, 0, 128), (32, 64, 16, 16, 1, 0, 128)]
    for it in range(12):
        if it < len(fixed) and dt == "fp16":
            Ci, Co, H, W, pu, pd, ns = fixed[it]
        else:
            Ci, Co = rng.choice([3, 8, 16, 24, 32, 64]), rng.choice([8, 16, 32, 40, 64])
            W = rng.choice([16, 32, 48] if dt == "fp16" else [8, 16, 24, 32])
            pu = rng.randint(0, 2)
            H = rng.randint(4, 33)
            pd = rng.randint(0, 2)
            if (H + pu + pd - 3) % 2:
                H += 1
            ns = rng.choice([1, 2, 5, 9, 32, 130])
        pl, pr = 1, 0  # (W + 1 + pr - 3) / 2 + 1 = W / 2 output columns with pr = 0 ... (W + pl + pr - 3) must be even
        if (W + pl + pr - 3) % 2:
            pr = 1
        Ho, Wo = (H + pu + pd - 3) // 2 + 1, (W + pl + pr - 3) // 2 + 1
        x = (torch.rand(ns, Ci, H, W, device="cuda") - 0.5).to(tdt)
        w = ((torch.rand(Co, Ci, 3, 3, device="cuda") - 0.5) * 0.5).to(tdt)
        dy = (torch.rand(ns, Co, Ho, Wo, device="cuda") - 0.5).to(tdt)
        y, dx, dw = torch.full_like(dy, 3), torch.full_like(x, 3), torch.full_like(w, 3)
        dx2, dw2 = torch.full_like(x, 3), torch.full_like(w, 3)
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, (pl, pr, pu, pd), (2, 2))
        a2, keep2 = hp.conv2d_args(pkg, x, dx2, w, dw2, y, dy, Ci, H, W, Co, 3, 3, Ho, Wo, (pl, pr, pu, pd), (2, 2))
        case = (Ci, Co, H, W, (pl, pr, pu, pd), ns)
        gpu.ptl_set_gemm_path(6)
        try:
            pkg.call("ptl_conv2d_%s_wg_batched" % dt, a, ns)
            if it < len(fixed) and dt == "fp16":
                assert gpu.ptl_last_conv_resident() == 2, case
            pkg.call("ptl_conv2d_%s_bw_batched" % dt, a2, ns)
        finally:
            gpu.ptl_set_gemm_path(0)
        gpu.ptl_sync()
        xp = F.pad(x.double(), (pl, pr, pu, pd))
        ref_dx = torch.nn.grad.conv2d_input(xp.shape, w.double(), dy.double(), stride=2)[:, :, pu:pu + H, pl:pl + W]
        ref_dw = torch.nn.grad.conv2d_weight(xp, w.shape, dy.double(), stride=2)
        assert rel(dw, ref_dw) <= tol, (case, "dw")
        assert rel(dx2, ref_dx) <= tol, (case, "dx, one call")
        assert rel(dw2, ref_dw) <= tol, (case, "dw, one call")


@pytest.mark.parametrize("dt,seed", [("fp16", 61), ("fp32", 62)])
def test_conv2d_small_layer_1x1_random_geometries(pkg, gpu, dt, seed):
    """1x1 layers without padding at stride 1 and 2 (the projection shortcuts of a ResNet: the small-layer kernels
    take them as a single tap, forced with path 6): forward, both gradients alone and in one call, against torch in
    float64."""
    rng = random.Random(seed)
    tdt, tol, vec = (torch.float16, 2e-3, 8) if dt == "fp16" else (torch.float32, 2e-5, 4)
    fixed = [(16, 32, 32, 2, 128), (32, 64, 16, 2, 128)]
    for it in range(12):
        if it < len(fixed):
            Ci, Co, H, st, ns = fixed[it]
            W = H
        else:
            Ci, Co = rng.choice([8, 16, 24, 32, 64]), rng.choice([8, 16, 32, 40, 64])
            st = rng.choice([1, 2])
            W = rng.choice([16, 32, 48] if dt == "fp16" else [8, 16, 24, 32])
            H = rng.randint(2, 33)
            ns = rng.choice([1, 2, 5, 9, 32, 130])
        Ho, Wo = (H - 1) // st + 1, (W - 1) // st + 1
        x = (torch.rand(ns, Ci, H, W, device="cuda") - 0.5).to(tdt)
        w = ((torch.rand(Co, Ci, 1, 1, device="cuda") - 0.5) * 0.5).to(tdt)
        dy = (torch.rand(ns, Co, Ho, Wo, device="cuda") - 0.5).to(tdt)
        y, dx, dw = torch.full_like(dy, 3), torch.full_like(x, 3), torch.full_like(w, 3)
        dx2, dw2 = torch.full_like(x, 3), torch.full_like(w, 3)
        # (a stride that does not divide the extent: the reference's naive-kernel route, USE_IM2COL = 0, takes it)
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, 1, 1, Ho, Wo, (0, 0, 0, 0), (st, st), 0, 1 if st == 1 else 0)
        a2, keep2 = hp.conv2d_args(pkg, x, dx2, w, dw2, y, dy, Ci, H, W, Co, 1, 1, Ho, Wo, (0, 0, 0, 0), (st, st), 0, 1 if st == 1 else 0)
        case = (Ci, Co, H, W, st, ns)
        gpu.ptl_set_gemm_path(6)
        try:
            for step, args in (("fw", a), ("wg", a), ("ig", a), ("bw", a2)):
                pkg.call("ptl_conv2d_%s_%s_batched" % (dt, step), args, ns)
                if it < len(fixed):
                    assert gpu.ptl_last_conv_resident() == 2, (case, step)
        finally:
            gpu.ptl_set_gemm_path(0)
        gpu.ptl_sync()
        ref_y = F.conv2d(x.double(), w.double(), stride=st)
        ref_dx = torch.nn.grad.conv2d_input(x.shape, w.double(), dy.double(), stride=st)
        ref_dw = torch.nn.grad.conv2d_weight(x.double(), w.shape, dy.double(), stride=st)
        assert rel(y, ref_y) <= tol, (case, "y")
        assert rel(dw, ref_dw) <= tol, (case, "dw")
        assert rel(dx, ref_dx) <= tol, (case, "dx")
        assert rel(dx2, ref_dx) <= tol, (case, "dx, one call")
        assert rel(dw2, ref_dw) <= tol, (case, "dw, one call")


@pytest.mark.parametrize("dt", ["fp16", "fp32"])
def test_conv2d_deferred_weight_gradient_sums(pkg, gpu, dt):
    """Backward calls that leave the addition of their partial sums to one flush: the same bits as the calls that add
    up themselves, for several layers in one batch (3x3 and 1x1, stride 1 and 2), a layer that does not take the
    small-layer kernels (completed by its own call), a batch too small for a layer (likewise) and an empty flush."""
    tdt = torch.float16 if dt == "fp16" else torch.float32
    layers = [(16, 16, 32, 3, 1, 128), (16, 32, 32, 3, 2, 128), (16, 32, 32, 1, 2, 128), (64, 64, 8, 3, 1, 130),
              (24, 40, 16, 3, 1, 5), (128, 128, 8, 3, 1, 4)]
    buf = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    for room in (buf.numel(), 600 << 10):
        batch = pkg.WgBatch()
        batch.buf, batch.bytes = buf.data_ptr(), room
        flush = getattr(gpu, "ptl_conv2d_%s_wg_flush" % dt)
        assert flush(ctypes.byref(batch)) == 0 and batch.count == 0, gpu.ptl_last_error()
        keep, pairs = [], []
        for (Ci, Co, H, k, st, ns) in layers:
            p = k // 2
            Ho = (H + 2 * p - k) // st + 1
            x = (torch.rand(ns, Ci, H, H, device="cuda") - 0.5).to(tdt)
            w = ((torch.rand(Co, Ci, k, k, device="cuda") - 0.5) * 0.5).to(tdt)
            dy = (torch.rand(ns, Co, Ho, Ho, device="cuda") - 0.5).to(tdt)
            y = torch.zeros_like(dy)
            outs = []
            for deferred in (False, True):
                dx, dw = torch.full_like(x, 3), torch.full_like(w, 3)
                a, kp = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, k, k, Ho, Ho, (p, p, p, p), (st, st), 0,
                                       1 if st == 1 else 0)
                keep.append((kp, x, w, dy, y))
                if deferred:
                    rc = getattr(gpu, "ptl_conv2d_%s_bw_batched_deferred" % dt)(ctypes.byref(a), ns, ctypes.byref(batch))
                    assert rc == 0, gpu.ptl_last_error()
                else:
                    pkg.call("ptl_conv2d_%s_bw_batched" % dt, a, ns)
                outs.append((dx, dw))
            pairs.append(outs)
        waiting = batch.count
        assert 0 < waiting < len(layers)  # (the 128-channel layer never waits; with little room fewer do)
        if room == buf.numel():  # (in fp32 a 64-channel tile can be too large for the small-layer kernels)
            assert waiting >= (len(layers) - 1 if dt == "fp16" else 3)
        assert flush(ctypes.byref(batch)) == 0, gpu.ptl_last_error()
        gpu.ptl_sync()
        assert batch.count == 0 and batch.used == 0
        for (now, later), layer in zip(pairs, layers):
            assert torch.equal(now[0], later[0]), (layer, "dx")
            assert torch.equal(now[1], later[1]), (layer, "dw")
    # tensors in host memory: the call works on staging copies that it copies back, so it completes the gradient
    # itself and leaves the batch alone
    nd = np.float16 if dt == "fp16" else np.float32
    Ci, Co, H, ns = 16, 16, 16, 8
    rng = np.random.default_rng(7)
    x, w, dy = [(rng.random(sh) - 0.5).astype(nd) for sh in ((ns, Ci, H, H), (Co, Ci, 3, 3), (ns, Co, H, H))]
    y = np.zeros_like(dy)
    host = []
    for deferred in (False, True):
        dx, dw = np.full_like(x, 3), np.full_like(w, 3)
        a, kp = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1), (1, 1))
        if deferred:
            assert getattr(gpu, "ptl_conv2d_%s_bw_batched_deferred" % dt)(ctypes.byref(a), ns, ctypes.byref(batch)) == 0
            assert batch.count == 0
        else:
            pkg.call("ptl_conv2d_%s_bw_batched" % dt, a, ns)
        host.append((dx, dw))
    assert np.array_equal(host[0][0], host[1][0]) and np.array_equal(host[0][1], host[1][1])


@pytest.mark.parametrize("dt", ["fp16", "fp32"])
def test_conv2d_deferred_weight_gradient_alone(pkg, gpu, dt):
    """A first layer has no input gradient: with skip_in_grad set the deferred backward call is the weight-gradient
    step alone, its sums wait for the flush like the others', and the result has the bits of ptl_conv2d_*_wg_batched."""
    tdt = torch.float16 if dt == "fp16" else torch.float32
    buf = torch.empty(8 << 20, dtype=torch.uint8, device="cuda")
    for (Ci, Co, H, ns) in ((3, 16, 32, 128), (16, 32, 16, 40)):
        x = (torch.rand(ns, Ci, H, H, device="cuda") - 0.5).to(tdt)
        w = (torch.rand(Co, Ci, 3, 3, device="cuda") - 0.5).to(tdt)
        dy = (torch.rand(ns, Co, H, H, device="cuda") - 0.5).to(tdt)
        y = torch.zeros_like(dy)
        outs = []
        for deferred in (False, True):
            dx, dw = torch.full_like(x, 3), torch.full_like(w, 3)
            a, kp = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1), (1, 1), 0, 1)
            a.skip_in_grad = 1
            if deferred:
                batch = pkg.WgBatch()
                batch.buf, batch.bytes = buf.data_ptr(), buf.numel()
                assert getattr(gpu, "ptl_conv2d_%s_bw_batched_deferred" % dt)(ctypes.byref(a), ns, ctypes.byref(batch)) == 0
                assert batch.count == 1
                assert getattr(gpu, "ptl_conv2d_%s_wg_flush" % dt)(ctypes.byref(batch)) == 0
            else:
                pkg.call("ptl_conv2d_%s_wg_batched" % dt, a, ns)
            assert gpu.ptl_sync() == 0
            assert bool((dx == 3).all())
            outs.append(dw)
        assert torch.equal(outs[0], outs[1]), (Ci, Co, H, ns)
        ref = torch.nn.grad.conv2d_weight(x.double(), w.shape, dy.double(), padding=1)
        assert rel(outs[1].double(), ref) <= (2e-3 if dt == "fp16" else 1e-5)


@pytest.mark.parametrize("dt", ["fp16", "fp32"])
def test_conv2d_forward_sums_feed_the_normalisation(pkg, gpu, dt):
    """ptl_conv2d_*_fw_batched_stats: the same output bits as the plain forward call, and per channel the sum of the
    output and of its squares (over the struct's parts, against the stored tensor summed in float64: the kernel sums
    its results before they are rounded to the tensor type, so in fp16 the two differ by the rounding noise of the
    elements, 2^-12 of the root of the sum of squares), for 3x3 and 1x1 layers, both strides, ragged last tiles and
    channel counts that do not fill a 32-filter block.  ptl_batch_norm_fused_*_fw_stats with them: the result of the
    call that forms its own sums to the rounding of the statistics.  Layers that cannot leave sums (a wide layer, one
    with a bias, a buffer that is too small) say so, and the normalisation then forms its own: bit for bit."""
    tdt = torch.float16 if dt == "fp16" else torch.float32
    tol_sum, tol_sq, tol_out = (2e-3, 1e-3, 1e-3) if dt == "fp16" else (2e-6, 1e-6, 1e-5)
    part = torch.empty(1 << 18, dtype=torch.float32, device="cuda")
    #        ns, Ci, Co, H, K, stride, bias, room in bytes, sums expected
    cases = [(128, 16, 16, 32, 3, 1, 0, part.numel() * 4, True), (128, 64, 64, 8, 3, 1, 0, part.numel() * 4, dt == "fp16"),
             (64, 16, 32, 32, 3, 2, 0, part.numel() * 4, True), (64, 16, 32, 32, 1, 2, 0, part.numel() * 4, True),
             (5, 24, 40, 16, 3, 1, 0, part.numel() * 4, True), (3, 8, 20, 24, 3, 1, 0, part.numel() * 4, True),
             (2, 3, 16, 32, 3, 1, 0, part.numel() * 4, True), (9, 64, 48, 8, 1, 1, 0, part.numel() * 4, True),
             (7, 12, 36, 24, 3, 1, 0, part.numel() * 4, True),
             (4, 128, 128, 8, 3, 1, 0, part.numel() * 4, False), (5, 24, 40, 16, 3, 1, 1, part.numel() * 4, False),
             (128, 16, 16, 32, 3, 1, 0, 4096, False)]
    for case in cases:
        ns, Ci, Co, H, K, s, bias, room, expect = case
        p = K // 2
        Ho = (H + 2 * p - K) // s + 1
        x = (torch.rand(ns, Ci, H, H, device="cuda") - 0.5).to(tdt)
        w = (torch.rand(Co, Ci, K, K, device="cuda") - 0.5).to(tdt)
        bs = (torch.rand(Co, device="cuda") - 0.5).to(tdt)
        y, y2 = torch.full((ns, Co, Ho, Ho), 3.0, device="cuda", dtype=tdt), torch.full((ns, Co, Ho, Ho), 3.0, device="cuda", dtype=tdt)
        part.fill_(7.0)
        st = pkg.NormStats()
        st.part, st.bytes, st.valid = part.data_ptr(), room, 5
        outs = []
        for out, with_sums in ((y, True), (y2, False)):
            a, kp = hp.conv2d_args(pkg, x, None, w, None, out, None, Ci, H, H, Co, K, K, Ho, Ho, (p, p, p, p), (s, s), 0,
                                   1 if s == 1 else 0, bs if bias else None)
            if with_sums:
                rc = getattr(gpu, "ptl_conv2d_%s_fw_batched_stats" % dt)(ctypes.byref(a), ns, ctypes.byref(st))
                assert rc == 0, gpu.ptl_last_error()
            else:
                pkg.call("ptl_conv2d_%s_fw_batched" % dt, a, ns)
        assert gpu.ptl_sync() == 0
        assert torch.equal(y, y2), case
        assert st.valid == (1 if expect else 0), case
        if st.valid:
            assert st.channels == Co and st.count == ns * Ho * Ho and st.parts >= 1
            used = Co * st.parts * 4
            assert used * 4 <= room and bool((part[used:] == 7.0).all()), case
            pt = part[:used].view(Co, st.parts, 4).double()
            s0, s1 = pt[:, :, 0].sum(1), pt[:, :, 1].sum(1)
            r0, r1 = y.double().sum((0, 2, 3)), (y.double() ** 2).sum((0, 2, 3))
            assert bool(((s0 - r0).abs() <= tol_sum * r1.sqrt()).all()), case
            assert bool(((s1 - r1).abs() <= tol_sq * r1).all()), case
        else:
            assert bool((part == 7.0).all()), case
        # the normalisation behind it, with a residual sum and a ReLU
        g, b = (torch.rand(Co, device="cuda") + 0.5).to(tdt), (torch.rand(Co, device="cuda") - 0.5).to(tdt)
        eps = torch.tensor([1e-5], device="cuda").to(tdt)
        skip = (torch.rand(ns, Co, Ho, Ho, device="cuda") - 0.5).to(tdt)
        o1, o2 = torch.full_like(y, 3), torch.full_like(y, 3)
        f = pkg.NormFusion()
        f.relu, f.skip = 1, skip.data_ptr()
        n1, k1 = hp.batch_norm_args(pkg, y, o1, g, b, eps, ns, Co, Ho, Ho)
        n2, k2 = hp.batch_norm_args(pkg, y, o2, g, b, eps, ns, Co, Ho, Ho)
        rc = getattr(gpu, "ptl_batch_norm_fused_%s_fw_stats" % dt)(ctypes.byref(n1), ctypes.byref(f), ctypes.byref(st))
        assert rc == 0, gpu.ptl_last_error()
        assert getattr(gpu, "ptl_batch_norm_fused_%s_fw" % dt)(ctypes.byref(n2), ctypes.byref(f)) == 0
        assert gpu.ptl_sync() == 0
        if st.valid:
            assert hp.rel_l2(o1.float().cpu().numpy(), o2.float().cpu().numpy()) <= tol_out, case
            # sums of another tensor (a count that does not match) are not taken
            st.count += 1
            o3 = torch.full_like(y, 3)
            n3, k3 = hp.batch_norm_args(pkg, y, o3, g, b, eps, ns, Co, Ho, Ho)
            assert getattr(gpu, "ptl_batch_norm_fused_%s_fw_stats" % dt)(ctypes.byref(n3), None, ctypes.byref(st)) == 0
            n4, k4 = hp.batch_norm_args(pkg, y, o2, g, b, eps, ns, Co, Ho, Ho)
            none = pkg.NormFusion()
            assert getattr(gpu, "ptl_batch_norm_fused_%s_fw" % dt)(ctypes.byref(n4), ctypes.byref(none)) == 0
            assert gpu.ptl_sync() == 0
            assert torch.equal(o3, o2), case  # (no fusion struct: nothing behind the normalisation)
        else:
            assert torch.equal(o1, o2), case


@pytest.mark.parametrize("dt", ["fp16", "fp32"])
def test_conv2d_forward_applies_the_normalisation_in_front(pkg, gpu, dt):
    """ptl_conv2d_*_fw_batched_normed against the two calls it stands for (ptl_batch_norm_fused_*_fw_stats, then
    ptl_conv2d_*_fw_batched_stats): the normalisation's output tensor, the convolution's output and the sums it
    leaves, bit for bit - where the small-layer kernel does both in one launch (ptl_last_conv_resident() == 3: 3x3
    layers of either stride with "same" padding, with and without ReLU and skip tensor, ragged tiles) and where it
    cannot and the two calls run (a wide layer, a strided 1x1 layer that does not read every row, no padding,
    sums that do not cover the tensor, host tensors); sums in 700 parts, more than a lane asks for early, are folded
    all the same."""
    tdt = torch.float16 if dt == "fp16" else torch.float32
    part0 = torch.empty(1 << 18, dtype=torch.float32, device="cuda")
    parts = [torch.empty(1 << 18, dtype=torch.float32, device="cuda") for _ in range(2)]
    #        ns, Cp, Ci, Co, H, K, stride, pad, relu, skip, sums valid, one launch expected (None: either)
    cases = [(128, 3, 16, 16, 32, 3, 1, 1, 1, 0, 1, True), (64, 16, 32, 32, 16, 3, 1, 1, 1, 1, 1, True),
             (32, 16, 16, 32, 32, 3, 2, 1, 1, 1, 1, True), (16, 32, 64, 64, 8, 3, 1, 1, 0, 1, 1, None),
             (5, 8, 24, 40, 16, 3, 1, 1, 1, 1, 1, None), (3, 8, 20, 12, 24, 3, 1, 1, 0, 0, 1, None),
             (7, 12, 36, 24, 24, 1, 1, 0, 1, 0, 1, None), (32, 16, 16, 32, 32, 1, 2, 0, 1, 1, 1, False),
             (8, 16, 16, 16, 16, 3, 1, 0, 1, 0, 1, False), (4, 16, 128, 128, 8, 3, 1, 1, 1, 1, 1, False),
             (64, 16, 32, 32, 16, 3, 1, 1, 1, 1, 0, False), (64, 16, 32, 32, 16, 3, 1, 1, 1, 1, 2, True)]
    fused = 0
    for case in cases:
        ns, Cp, Ci, Co, H, K, s, p, relu, with_skip, sums_valid, expect = case
        Ho = (H + 2 * p - K) // s + 1
        # the layer in front: a 3x3 convolution whose output the normalisation reads, and its sums
        xp = (torch.rand(ns, Cp, H, H, device="cuda") - 0.5).to(tdt)
        wp = (torch.rand(Ci, Cp, 3, 3, device="cuda") - 0.5).to(tdt)
        y0 = torch.zeros(ns, Ci, H, H, device="cuda", dtype=tdt)
        a0, k0 = hp.conv2d_args(pkg, xp, None, wp, None, y0, None, Cp, H, H, Ci, 3, 3, H, H, (1, 1, 1, 1), (1, 1), 0, 1)
        st_in = pkg.NormStats()
        st_in.part, st_in.bytes = part0.data_ptr(), part0.numel() * 4
        assert getattr(gpu, "ptl_conv2d_%s_fw_batched_stats" % dt)(ctypes.byref(a0), ns, ctypes.byref(st_in)) == 0
        if not st_in.valid:  # (a layer in front that leaves no sums: those of the stored tensor, as one part)
            part0[:Ci * 4].view(Ci, 1, 4)[:, 0, 0] = y0.double().sum((0, 2, 3)).float()
            part0[:Ci * 4].view(Ci, 1, 4)[:, 0, 1] = (y0.double() ** 2).sum((0, 2, 3)).float()
            st_in.count, st_in.parts, st_in.channels, st_in.valid = ns * H * H, 1, Ci, 1
        if not sums_valid:
            st_in.count += 1
        if sums_valid == 2:  # (more parts than a lane asks for early: 700, the sums spread over them)
            np_ = 700
            sums = torch.stack((y0.double().sum((0, 2, 3)), (y0.double() ** 2).sum((0, 2, 3))), 1)  # [Ci][2]
            wgt = torch.rand(Ci, np_, 1, device="cuda", dtype=torch.float64)
            wgt = wgt / wgt.sum(1, keepdim=True)
            pv = part0[:Ci * np_ * 4].view(Ci, np_, 4)
            pv.zero_()
            pv[:, :, :2] = (wgt * sums[:, None, :]).float()
            st_in.count, st_in.parts, st_in.channels, st_in.valid = ns * H * H, np_, Ci, 1
        gm, bt = (torch.rand(Ci, device="cuda") + 0.5).to(tdt), (torch.rand(Ci, device="cuda") - 0.5).to(tdt)
        eps = torch.tensor([1e-5], device="cuda").to(tdt)
        skip = (torch.rand(ns, Ci, H, H, device="cuda") - 0.5).to(tdt)
        w = (torch.rand(Co, Ci, K, K, device="cuda") - 0.5).to(tdt)
        f = pkg.NormFusion()
        f.relu, f.skip = relu, skip.data_ptr() if with_skip else None
        res = []
        for one_call in (False, True):
            out, y = torch.full_like(y0, 3), torch.full((ns, Co, Ho, Ho), 3.0, device="cuda", dtype=tdt)
            na, kn = hp.batch_norm_args(pkg, y0, out, gm, bt, eps, ns, Ci, H, H)
            a, kp = hp.conv2d_args(pkg, out, None, w, None, y, None, Ci, H, H, Co, K, K, Ho, Ho, (p, p, p, p), (s, s), 0,
                                   1 if s == 1 else 0)
            st = pkg.NormStats()
            parts[one_call].fill_(7.0)
            st.part, st.bytes = parts[one_call].data_ptr(), parts[one_call].numel() * 4
            if one_call:
                rc = getattr(gpu, "ptl_conv2d_%s_fw_batched_normed" % dt)(ctypes.byref(a), ns, ctypes.byref(st), ctypes.byref(na),
                                                                         ctypes.byref(f), ctypes.byref(st_in))
                assert rc == 0, gpu.ptl_last_error()
                took = gpu.ptl_last_conv_resident() == 3
            else:
                assert getattr(gpu, "ptl_batch_norm_fused_%s_fw_stats" % dt)(ctypes.byref(na), ctypes.byref(f), ctypes.byref(st_in)) == 0
                assert getattr(gpu, "ptl_conv2d_%s_fw_batched_stats" % dt)(ctypes.byref(a), ns, ctypes.byref(st)) == 0
            assert gpu.ptl_sync() == 0
            res.append((out, y, st))
        (out_a, y_a, st_a), (out_b, y_b, st_b) = res
        assert expect is None or took == expect, case
        fused += took
        assert torch.equal(out_a, out_b), case
        assert torch.equal(y_a, y_b), case
        assert (st_a.valid, st_a.parts, st_a.channels, st_a.count) == (st_b.valid, st_b.parts, st_b.channels, st_b.count), case
        assert torch.equal(parts[0], parts[1]), case
    assert fused >= 4
    # host tensors: the two calls, staged
    xh = hp.uniform(5, (2, 16, 8, 8), -0.5, 0.5).astype(hp.np_dtype(dt))
    wh = hp.uniform(6, (16, 16, 3, 3), -0.5, 0.5).astype(xh.dtype)
    gh, bh, eh = np.ones(16, xh.dtype), np.zeros(16, xh.dtype), np.full(1, 1e-5, xh.dtype)
    outs = []
    for one_call in (False, True):
        oh, yh = np.zeros_like(xh), np.zeros((2, 16, 8, 8), xh.dtype)
        na, kn = hp.batch_norm_args(pkg, xh, oh, gh, bh, eh, 2, 16, 8, 8)
        a, kp = hp.conv2d_args(pkg, oh, None, wh, None, yh, None, 16, 8, 8, 16, 3, 3, 8, 8, (1, 1, 1, 1), (1, 1), 0, 1)
        none = pkg.NormFusion()
        if one_call:
            assert getattr(gpu, "ptl_conv2d_%s_fw_batched_normed" % dt)(ctypes.byref(a), 2, None, ctypes.byref(na), ctypes.byref(none), None) == 0
        else:
            assert getattr(gpu, "ptl_batch_norm_fused_%s_fw" % dt)(ctypes.byref(na), ctypes.byref(none)) == 0
            pkg.call("ptl_conv2d_%s_fw_batched" % dt, a, 2)
        outs.append((oh, yh))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
    assert np.abs(outs[0][1]).max() > 0


@pytest.mark.parametrize("dt", ["fp16", "fp32"])
def test_conv2d_backward_forms_the_gradient_of_the_normalisation_in_front(pkg, gpu, dt):
    """ptl_conv2d_*_bw_batched_deferred_post: where the small-layer kernel takes the layer (sums.valid == 1), input->diff
    is bit for bit what the plain call's input gradient, the addition of a second gradient (rounded to the tensor type)
    and the ReLU mask give as separate steps, the weight gradient is the plain call's, and the struct's parts add up to
    the sums of that gradient and of its products with the normalisation's input (float64 sums of the stored tensors;
    the kernel adds the same values in fp32).  Elsewhere input->diff is the plain input gradient and nothing is
    written to the buffer.  ptl_batch_norm_fused_*_bw_stats behind it: against ptl_batch_norm_fused_*_bw on the
    plain gradient with the same addition and mask, to the rounding of the statistics - with the forward sums given
    (one launch) and without (two), and bit for bit when the convolution left no sums."""
    tdt = torch.float16 if dt == "fp16" else torch.float32
    tol = 2e-3 if dt == "fp16" else 2e-5
    part = torch.empty(1 << 18, dtype=torch.float32, device="cuda")
    wg_buf = torch.empty(16 << 20, dtype=torch.uint8, device="cuda")
    #        ns, Ci, Co, H, K, stride, add, mask, room, sums expected (None: either)
    room = part.numel() * 4
    cases = [(128, 16, 16, 32, 3, 1, 1, 1, room, True), (64, 32, 32, 16, 3, 1, 0, 1, room, True),
             (32, 64, 64, 8, 3, 1, 1, 0, room, None), (64, 16, 32, 16, 3, 1, 1, 1, room, True),
             (5, 24, 40, 16, 3, 1, 1, 1, room, None), (3, 8, 20, 24, 3, 1, 0, 0, room, None),
             (7, 12, 36, 24, 3, 1, 1, 1, room, None), (64, 16, 32, 32, 3, 2, 1, 1, room, None),
             (4, 128, 128, 8, 3, 1, 1, 1, room, False), (128, 16, 16, 32, 3, 1, 1, 1, 4096, False)]
    taken = 0
    for case in cases:
        ns, Ci, Co, H, K, s, with_add, with_mask, room, expect = case
        p = K // 2
        Ho = (H + 2 * p - K) // s + 1
        x = (torch.rand(ns, Ci, H, H, device="cuda") - 0.5).to(tdt)
        w = (torch.rand(Co, Ci, K, K, device="cuda") - 0.5).to(tdt)
        dy = (torch.rand(ns, Co, Ho, Ho, device="cuda") - 0.5).to(tdt)
        y = torch.zeros(ns, Co, Ho, Ho, device="cuda", dtype=tdt)
        add = (torch.rand(ns, Ci, H, H, device="cuda") - 0.5).to(tdt)
        xn = (torch.rand(ns, Ci, H, H, device="cuda") - 0.3).to(tdt)  # the normalisation's input; x is its output
        got = []
        for post_mode in (False, True):
            dx, dw = torch.full_like(x, 3), torch.full_like(w, 3)
            a, kp = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, K, K, Ho, Ho, (p, p, p, p), (s, s), 0,
                                   1 if s == 1 else 0)
            batch = pkg.WgBatch()
            batch.buf, batch.bytes = wg_buf.data_ptr(), wg_buf.numel()
            st = pkg.NormStats()
            part.fill_(7.0)
            st.part, st.bytes, st.valid = part.data_ptr(), room, 5
            if post_mode:
                po = pkg.GradPost()
                po.add, po.mask, po.x = add.data_ptr() if with_add else None, x.data_ptr() if with_mask else None, xn.data_ptr()
                rc = getattr(gpu, "ptl_conv2d_%s_bw_batched_deferred_post" % dt)(ctypes.byref(a), ns, ctypes.byref(batch),
                                                                                ctypes.byref(po), ctypes.byref(st))
            else:
                rc = getattr(gpu, "ptl_conv2d_%s_bw_batched_deferred" % dt)(ctypes.byref(a), ns, ctypes.byref(batch))
            assert rc == 0, gpu.ptl_last_error()
            assert getattr(gpu, "ptl_conv2d_%s_wg_flush" % dt)(ctypes.byref(batch)) == 0
            assert gpu.ptl_sync() == 0
            got.append((dx, dw, st))
        (dx0, dw0, _), (dx1, dw1, st) = got
        assert torch.equal(dw0, dw1), case
        assert st.valid in (0, 1) and (expect is None or st.valid == int(expect)), case
        g_ref = dx0
        if with_add:
            g_ref = (g_ref.float() + add.float()).to(tdt)
        if with_mask:
            g_ref = torch.where(x > 0, g_ref, torch.zeros_like(g_ref))
        if st.valid:
            taken += 1
            assert torch.equal(dx1, g_ref), case
            assert st.channels == Ci and st.count == ns * H * H and st.parts >= 1
            used = Ci * st.parts * 4
            assert used * 4 <= room and bool((part[used:] == 7.0).all()), case
            pt = part[:used].view(Ci, st.parts, 4).double()
            s0, s1 = pt[:, :, 0].sum(1), pt[:, :, 1].sum(1)
            gd, xd = g_ref.double(), xn.double()
            r0, r1 = gd.sum((0, 2, 3)), (gd * xd).sum((0, 2, 3))
            assert bool(((s0 - r0).abs() <= 1e-5 * gd.abs().sum((0, 2, 3)) + 1e-6).all()), case
            assert bool(((s1 - r1).abs() <= 1e-5 * (gd * xd).abs().sum((0, 2, 3)) + 1e-6).all()), case
        else:
            assert torch.equal(dx1, dx0), case
            assert bool((part == 7.0).all()), case
        # the normalisation in front of the convolution: input xn, output x (the mask), gradient of the output dx
        gm, bt = (torch.rand(Ci, device="cuda") + 0.5).to(tdt), (torch.rand(Ci, device="cuda") - 0.5).to(tdt)
        eps = torch.tensor([1e-5], device="cuda").to(tdt)
        fw_part = torch.zeros(Ci, 1, 4, dtype=torch.float32, device="cuda")
        fw_part[:, 0, 0], fw_part[:, 0, 1] = xn.double().sum((0, 2, 3)).float(), (xn.double() ** 2).sum((0, 2, 3)).float()
        fw = pkg.NormStats()
        fw.part, fw.bytes, fw.count, fw.parts, fw.channels, fw.valid = fw_part.data_ptr(), fw_part.numel() * 4, ns * H * H, 1, Ci, 1
        # the reference: the fused backward call on the plain gradient
        dyr, dxr, dgr, dbr = dx0.clone(), torch.full_like(x, 3), torch.full_like(gm, 3), torch.full_like(gm, 3)
        fr = pkg.NormFusion()
        fr.relu, fr.diff2, fr.skip_diff = with_mask, add.data_ptr() if with_add else None, dyr.data_ptr()
        nr, kr = hp.batch_norm_args(pkg, xn, x, gm, bt, eps, ns, Ci, H, H, dxr, dyr, dgr, dbr)
        assert getattr(gpu, "ptl_batch_norm_fused_%s_bw" % dt)(ctypes.byref(nr), ctypes.byref(fr)) == 0
        assert gpu.ptl_sync() == 0
        assert torch.equal(dyr, g_ref), case  # (the gradient of the sum, in place)
        for fw_given in (fw, None):
            dyn, dxn, dgn, dbn = dx1.clone(), torch.full_like(x, 3), torch.full_like(gm, 3), torch.full_like(gm, 3)
            fn = pkg.NormFusion()
            fn.relu, fn.diff2, fn.skip_diff = with_mask, add.data_ptr() if with_add else None, dyn.data_ptr()
            nn_, kn = hp.batch_norm_args(pkg, xn, x, gm, bt, eps, ns, Ci, H, H, dxn, dyn, dgn, dbn)
            rc = getattr(gpu, "ptl_batch_norm_fused_%s_bw_stats" % dt)(ctypes.byref(nn_), ctypes.byref(fn),
                                                                      ctypes.byref(fw_given) if fw_given else None, ctypes.byref(st))
            assert rc == 0, gpu.ptl_last_error()
            assert gpu.ptl_sync() == 0
            assert torch.equal(dyn, g_ref), case
            if st.valid:
                assert hp.rel_l2(dxn.float().cpu().numpy(), dxr.float().cpu().numpy()) <= tol, case
                assert hp.rel_l2(dgn.float().cpu().numpy(), dgr.float().cpu().numpy()) <= tol, case
                assert hp.rel_l2(dbn.float().cpu().numpy(), dbr.float().cpu().numpy()) <= tol, case
            else:
                assert torch.equal(dxn, dxr) and torch.equal(dgn, dgr) and torch.equal(dbn, dbr), case
    assert taken >= 3
    # host tensors are rejected
    xh = np.zeros((2, 16, 8, 8), dtype=hp.np_dtype(dt))
    wh, yh = np.zeros((16, 16, 3, 3), dtype=xh.dtype), np.zeros((2, 16, 8, 8), dtype=xh.dtype)
    a, kp = hp.conv2d_args(pkg, xh, xh.copy(), wh, wh.copy(), yh, yh.copy(), 16, 8, 8, 16, 3, 3, 8, 8, (1, 1, 1, 1), (1, 1), 0, 1)
    po, st = pkg.GradPost(), pkg.NormStats()
    po.x = xh.ctypes.data
    rc = getattr(gpu, "ptl_conv2d_%s_bw_batched_deferred_post" % dt)(ctypes.byref(a), 2, None, ctypes.byref(po), ctypes.byref(st))
    assert rc == 1 and st.valid == 0


@pytest.mark.parametrize("seed", [21, 22])
def test_depthwise_random_geometries(pkg, gpu, seed):
    rng = random.Random(seed)
    for it in range(14):
        C, ns = rng.choice([32, 64, 96]), rng.choice([8, 16, 24])
        pl, pr, pu, pd = rng.choice([0, 2]), rng.randint(0, 2), rng.randint(0, 2), rng.randint(0, 2)
        W, H = rng.choice([30, 32, 34, 40, 46, 56, 58, 64]), rng.randint(8, 60)
        Ho, Wo = H + pu + pd - 2, W + pl + pr - 2
        x = (torch.rand(ns, C, H, W, device="cuda") - 0.5).half()
        w = (torch.rand(C, 3, 3, device="cuda") - 0.5).half()
        dy = (torch.rand(ns, C, Ho, Wo, device="cuda") - 0.5).half()
        y, dx, dw = torch.full_like(dy, 3), torch.full_like(x, 3), torch.full_like(w, 3)
        a, keep = hp.dw_args(pkg, "fp16", x, dx, w, dw, y, dy, C, H, W, 3, 3, Ho, Wo, (pl, pr, pu, pd))
        for s in ("fw", "wg", "ig"):
            pkg.call("ptl_conv_dw_fp16_%s_batched" % s, a, ns)
        gpu.ptl_sync()
        xp = F.pad(x.float(), (pl, pr, pu, pd)).requires_grad_(True)
        wf = w.float().unsqueeze(1).requires_grad_(True)
        ref_y = F.conv2d(xp, wf, groups=C)
        ref_y.backward(dy.float())
        case = (C, H, W, (pl, pr, pu, pd), ns)
        assert rel(y, ref_y.detach()) <= 2e-3, (case, "y")
        assert rel(dw, wf.grad.squeeze(1)) <= 2e-3, (case, "dw")
        assert rel(dx, xp.grad[:, :, pu:pu + H, pl:pl + W]) <= 2e-3, (case, "dx")
