"""The allocation-free depthwise weight gradient (ptl_conv_dw_fp16_wg_noalloc) against the allocating entry point
it mirrors (ptl_conv_dw_fp16_wg_batched): same kernels, so the results must be bit-identical; two calls in a row
on the shared fixed buffer, the second on a smaller input; rejections leave the output untouched."""
import numpy as np
import pytest
import torch

import helpers as hp

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def both(pkg, gpu, C, H, W, K, ns, seed):
    Ho, Wo = H - K + 1, W - K + 1
    x = dev(hp.uniform(seed, (ns, C, H, W), dtype=np.float16))
    dy = dev(hp.uniform(seed + 1, (ns, C, Ho, Wo), dtype=np.float16))
    out = []
    for name in ("ptl_conv_dw_fp16_wg_batched", "ptl_conv_dw_fp16_wg_noalloc"):
        dw = dev(np.full((C, K, K), 3, np.float16))
        a, keep = hp.dw_args(pkg, "fp16", x, None, None, dw, None, dy, C, H, W, K, K, Ho, Wo)
        pkg.call(name, a, ns)
        assert gpu.ptl_sync() == 0, gpu.ptl_last_error().decode()
        out.append(dw.cpu().numpy())
    ref = torch.nn.grad.conv2d_weight(x.float().reshape(1, ns * C, H, W), (ns * C, 1, K, K),
                                      dy.float().reshape(1, ns * C, Ho, Wo), groups=ns * C)
    ref = ref.reshape(ns, C, K, K).sum(0).cpu().numpy()
    return out[0], out[1], ref


def test_noalloc_depthwise_weight_gradient_matches_allocating_entry_point(pkg, gpu):
    # BASELINE config 3 at batch 64 (plane-resident kernels, 16 sample groups of partial sums) ...
    a, b, ref = both(pkg, gpu, 64, 58, 58, 3, 64, 0xC0DE0701)
    assert np.array_equal(a, b)
    assert hp.rel_l2(b, ref) <= 1e-3
    # ... then a smaller input on the same fixed buffer (fewer groups: stale partial sums must not be read)
    a, b, ref = both(pkg, gpu, 16, 36, 36, 3, 40, 0xC0DE0702)
    assert np.array_equal(a, b)
    assert hp.rel_l2(b, ref) <= 1e-3
    # the other kernel families: rows wider than a plane-resident tile, a 5x5 filter, the generic geometry
    for case in ((8, 150, 160, 3, 6), (32, 38, 40, 5, 16), (5, 9, 11, 3, 3), (24, 40, 40, 3, 1)):
        a, b, ref = both(pkg, gpu, *case, 0xC0DE0703)
        assert np.array_equal(a, b), case
        assert hp.rel_l2(b, ref) <= 1e-3, case


def test_noalloc_entry_point_called_first_allocates_no_device_memory(pkg, gpu):
    """The allocation-free entry point on a geometry that no allocating call has prepared: free device memory is
    the same before and after, the result is right, and only then the allocating twin runs (bit-identical)."""
    C, H, W, K, ns = 20, 44, 52, 3, 7
    Ho, Wo = H - K + 1, W - K + 1
    x = dev(hp.uniform(0xC0DE0710, (ns, C, H, W), dtype=np.float16))
    dy = dev(hp.uniform(0xC0DE0711, (ns, C, Ho, Wo), dtype=np.float16))
    dw = dev(np.full((C, K, K), 3, np.float16))
    dw2 = dev(np.full((C, K, K), 3, np.float16))
    ref = torch.nn.grad.conv2d_weight(x.float().reshape(1, ns * C, H, W), (ns * C, 1, K, K),
                                      dy.float().reshape(1, ns * C, Ho, Wo), groups=ns * C)
    ref = ref.reshape(ns, C, K, K).sum(0).cpu().numpy()
    a, keep = hp.dw_args(pkg, "fp16", x, None, None, dw, None, dy, C, H, W, K, K, Ho, Wo)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    pkg.call("ptl_conv_dw_fp16_wg_noalloc", a, ns)
    assert gpu.ptl_sync() == 0, gpu.ptl_last_error().decode()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    assert hp.rel_l2(dw.cpu().numpy(), ref) <= 1e-3
    a2, keep2 = hp.dw_args(pkg, "fp16", x, None, None, dw2, None, dy, C, H, W, K, K, Ho, Wo)
    pkg.call("ptl_conv_dw_fp16_wg_batched", a2, ns)
    assert gpu.ptl_sync() == 0
    assert torch.equal(dw, dw2)


def test_noalloc_rejections_leave_the_output_untouched(pkg, gpu):
    C, H, K, ns = 8, 12, 3, 2
    x = hp.uniform(1, (ns, C, H, H), dtype=np.float16)
    dy = dev(hp.uniform(2, (ns, C, H - K + 1, H - K + 1), dtype=np.float16))
    dw = dev(np.full((C, K, K), 3, np.float16))
    # a host pointer would need a staging buffer
    a, keep = hp.dw_args(pkg, "fp16", x, None, None, dw, None, dy, C, H, H, K, K, H - K + 1, H - K + 1)
    with pytest.raises(RuntimeError, match="may not allocate"):
        pkg.call("ptl_conv_dw_fp16_wg_noalloc", a, ns)
    # partial sums beyond the fixed buffer: 8192 channels x 49 taps x 4 bytes = 1.5 MiB
    C2, K2 = 8192, 7
    x2 = dev(np.zeros((1, C2, K2, K2), np.float16))
    dy2 = dev(np.zeros((1, C2, 1, 1), np.float16))
    dw2 = dev(np.full((C2, K2, K2), 3, np.float16))
    a2, keep2 = hp.dw_args(pkg, "fp16", x2, None, None, dw2, None, dy2, C2, K2, K2, K2, K2, 1, 1)
    with pytest.raises(RuntimeError, match="fixed buffer"):
        pkg.call("ptl_conv_dw_fp16_wg_noalloc", a2, 1)
    assert gpu.ptl_sync() == 0
    assert torch.all(dw == 3) and torch.all(dw2 == 3)
    # the allocating entry point takes the same call
    pkg.call("ptl_conv_dw_fp16_wg_batched", a2, 1)
    assert gpu.ptl_sync() == 0
    assert torch.all(dw2 == 0)
