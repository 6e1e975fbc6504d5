"""Which kernel family the default selection (ptl_set_gemm_path(0)) gives the 3x3 fp16 Conv2D shapes that bench.py
times, step by step.  The families are chosen by measured thresholds in the launchers; a change that moves one of
these shapes to another family by accident shows here, not as a slower row in the next benchmark.

ptl_last_conv_resident(): 1 = input tile resident in LDS for all taps (wide layers), 2 = small-layer kernel, 0 = other;
ptl_last_conv_direct(): 1 = a convolution kernel or the tap-sum product, 0 = the implicit-im2col GEMM."""
import ctypes

import pytest
import torch

import helpers as hp

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# (HWC, batch, Cin, Cout, H = W, [(resident, direct) after FW, WG, IG])
TABLE = [
    (0, 128, 16, 32, 32, [(2, 1), (2, 1), (2, 1)]),    # BASELINE config 1 in fp16, batched
    (0, 1, 16, 32, 32, [(2, 1), (0, 1), (2, 1)]),      # ... one sample
    (0, 128, 16, 16, 32, [(2, 1), (2, 1), (2, 1)]),    # ResNet-20 stage 1
    (0, 128, 64, 64, 8, [(2, 1), (2, 1), (2, 1)]),     # ResNet-20 stage 3
    (0, 256, 32, 64, 56, [(2, 1), (0, 1), (1, 1)]),    # input gradient: 64 channels into 32-filter resident tiles
    (0, 128, 64, 64, 56, [(1, 1), (0, 1), (1, 1)]),    # 64 filters: the weight gradient's resident-tile kernel needs 128
    (0, 64, 128, 128, 56, [(1, 1), (1, 1), (1, 1)]),   # rows 57 wide: four pieces of the input tile per unit of the weight gradient
    (0, 128, 128, 128, 28, [(1, 1), (1, 1), (1, 1)]),
    (0, 128, 256, 256, 14, [(1, 1), (1, 1), (1, 1)]),
    (0, 512, 128, 128, 28, [(1, 1), (1, 1), (1, 1)]),
    (0, 256, 256, 256, 28, [(1, 1), (1, 1), (1, 1)]),
    (0, 256, 512, 512, 14, [(1, 1), (1, 1), (1, 1)]),
    (1, 128, 64, 64, 56, [(1, 1), (1, 1), (1, 1)]),    # channel-minor: all three steps on the caller's tensors in place
    (1, 128, 128, 128, 28, [(1, 1), (1, 1), (1, 1)]),
    (1, 128, 256, 256, 14, [(1, 1), (1, 1), (1, 1)]),
    (0, 8, 128, 128, 28, [(0, 1), (1, 1), (0, 1)]),    # too few tiles for the persistent forward kernel; the weight
                                                       # gradient's resident-tile kernel pays from 48 units of positions
    (1, 8, 128, 128, 28, [(0, 1), (1, 1), (0, 1)]),
]


@pytest.mark.parametrize("row", TABLE)
def test_default_route_of_bench_shapes(pkg, gpu, row):
    hwc, ns, Ci, Co, H, want = row
    g = torch.Generator(device="cpu").manual_seed(3)
    x = (torch.rand(ns, Ci, H, H, generator=g) - 0.5).half().to(DEV)
    w = ((torch.rand(Co, Ci, 3, 3, generator=g) - 0.5) * 0.2).half().to(DEV)
    dy = (torch.rand(ns, Co, H, H, generator=g) - 0.5).half().to(DEV)
    if hwc:
        x, w, dy = [t.permute(0, 2, 3, 1).contiguous() for t in (x, w, dy)]
    y, dx, dw = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
    a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1), (1, 1), hwc)
    gpu.ptl_set_gemm_path(0)
    got = []
    for s in ("fw", "wg", "ig"):
        assert getattr(gpu, "ptl_conv2d_fp16_%s_batched" % s)(ctypes.byref(a), ns) == 0, gpu.ptl_last_error().decode()
        got.append((gpu.ptl_last_conv_resident(), gpu.ptl_last_conv_direct()))
    assert gpu.ptl_sync() == 0
    assert got == want
    # and whatever the route, the forward result of the first samples is right
    n = min(ns, 4)
    cm = (lambda t: t.permute(0, 3, 1, 2)) if hwc else (lambda t: t)
    ref = torch.nn.functional.conv2d(cm(x[:n].float()), cm(w.float()), padding=1)
    assert float((cm(y[:n].float()) - ref).norm() / ref.norm()) <= 1e-3


@pytest.mark.parametrize("case", [(8, 512, 512, 14, 0), (24, 256, 256, 14, 1), (8, 128, 128, 28, 0), (12, 128, 128, 28, 1)])
def test_one_call_backward_takes_the_pair_only_with_tiles_enough(pkg, gpu, case):
    """ptl_conv2d_fp16_bw_batched: weight and input gradient share the blocked copy of the output gradient between the
    two resident-tile kernels only where the input gradient's persistent kernel has 40 tiles and more; below that the
    call does the two single steps (the last of which, the input gradient, is then no resident-tile launch).  Same
    bits as the two single calls either way."""
    ns, Ci, Co, H, pair = case
    g = torch.Generator(device="cpu").manual_seed(5)
    x = (torch.rand(ns, Ci, H, H, generator=g) - 0.5).half().to(DEV)
    w = ((torch.rand(Co, Ci, 3, 3, generator=g) - 0.5) * 0.2).half().to(DEV)
    dy = (torch.rand(ns, Co, H, H, generator=g) - 0.5).half().to(DEV)
    dx, dw = torch.zeros_like(x), torch.zeros_like(w)
    a, keep = hp.conv2d_args(pkg, x, dx, w, dw, None, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1), (1, 1))
    gpu.ptl_set_gemm_path(0)
    assert gpu.ptl_conv2d_fp16_bw_batched(ctypes.byref(a), ns) == 0, gpu.ptl_last_error().decode()
    assert gpu.ptl_last_conv_resident() == pair
    assert gpu.ptl_sync() == 0
    dx2, dw2 = torch.zeros_like(x), torch.zeros_like(w)
    b, keep2 = hp.conv2d_args(pkg, x, dx2, w, dw2, None, dy, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1), (1, 1))
    assert gpu.ptl_conv2d_fp16_wg_batched(ctypes.byref(b), ns) == 0
    assert gpu.ptl_conv2d_fp16_ig_batched(ctypes.byref(b), ns) == 0
    assert gpu.ptl_sync() == 0
    assert torch.equal(dw2, dw)
    ref = torch.nn.grad.conv2d_input(x.shape, w.float(), dy.float(), padding=1)
    for t in (dx, dx2):
        assert float((t.float() - ref).norm() / ref.norm()) <= 2e-3
