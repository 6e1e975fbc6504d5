"""The index helpers at the sizes the benchmark times them on (64 MiB and more), bit-exact against the same
permutation written with torch's own indexing operations on the device: the small geometries of the parity tests
leave the many-workgroup paths (tile groups, several sweeps of a row, the last partial piece of a large tensor)
to these."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import helpers as hp

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TDT = {"fp32": torch.float32, "fp16": torch.float16}


def sync(lib):
    assert lib.ptl_sync() == 0, lib.ptl_last_error().decode()


def same_bits(a, b):
    it = torch.int32 if a.dtype == torch.float32 else torch.int16
    return bool(torch.equal(a.contiguous().view(it), b.contiguous().view(it)))


def payload(n, dt, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.rand(n, device=DEV, generator=g) - 0.5).to(TDT[dt])


@pytest.mark.parametrize("dt,Ci,H,W,K,pad", [("fp16", 64, 224, 224, 3, 1), ("fp32", 64, 224, 224, 3, 1),
                                            ("fp16", 24, 150, 200, 5, 2), ("fp16", 20, 96, 100, 3, 1)])
def test_im2row_and_im2col_of_a_large_plane(pkg, gpu, dt, Ci, H, W, K, pad):
    x = payload(Ci * H * W, dt, 5).view(Ci, H, W)
    Ho, Wo = H + 2 * pad - K + 1, W + 2 * pad - K + 1
    n = Ho * Wo * Ci * K * K
    bi, bw, bo = pkg.blob(x, None, Ci, H, W), pkg.blob(None, None, Ci, K, K), pkg.blob(None, None, 1, Ho, Wo)
    a = pkg.Im2colArgs()
    a.input, a.c, a.output = hp.ptr(bi), hp.ptr(bw), hp.ptr(bo)
    a.Lpad = a.Rpad = a.Upad = a.Dpad = pad
    a.stride_h = a.stride_w = 1
    # unfold: [Ci*K*K, Ho*Wo] with rows (c, hk, wk) - the column-major patch matrix; its transpose is the row-major one
    cols = F.unfold(x.float().unsqueeze(0), K, padding=pad)[0].to(TDT[dt])
    for fn, ref in (("im2row", cols.t().contiguous()), ("im2col", cols)):
        buf = torch.full((n + 8,), 7.0, device=DEV, dtype=TDT[dt])
        a.pBuffer = buf.data_ptr()
        pkg.call("pulp_%s_%s" % (fn, dt), a)
        sync(gpu)
        assert same_bits(buf[:n], ref.reshape(-1)), fn
        assert bool((buf[n:] == 7.0).all()), fn + " wrote behind its buffer"


@pytest.mark.parametrize("dt,Ci,Co", [("fp16", 2048, 2048), ("fp16", 1000, 520), ("fp32", 640, 768)])
def test_blocktranspose_of_large_filter_banks(pkg, gpu, dt, Ci, Co):
    w = payload(Co * Ci * 9, dt, 6).view(Co, Ci, 9)
    out = torch.full((Co * Ci * 9 + 8,), 7.0, device=DEV, dtype=TDT[dt])
    a = pkg.BlocktranspArgs()
    a.weights, a.bt_weights, a.Cin, a.Cout, a.Hk, a.Wk, a.HWC = w.data_ptr(), out.data_ptr(), Ci, Co, 3, 3, 0
    pkg.call("pulp_blocktransp_" + dt, a)
    sync(gpu)
    ref = w.flip(2).permute(1, 0, 2).contiguous()
    assert same_bits(out[:Co * Ci * 9], ref.reshape(-1))
    assert bool((out[Co * Ci * 9:] == 7.0).all())


@pytest.mark.parametrize("dt,hwc,C,H,W,pads", [("fp16", 0, 256, 360, 360, (1, 1, 1, 1)), ("fp16", 1, 64, 300, 301, (2, 0, 1, 3)),
                                              ("fp32", 0, 96, 250, 123, (0, 3, 2, 1)), ("fp16", 0, 3, 2000, 3001, (1, 2, 0, 1))])
def test_pad_of_large_tensors(pkg, gpu, dt, hwc, C, H, W, pads):
    L, R, U, D = pads
    x = payload(C * H * W, dt, 7).view(C, H, W)
    ref = F.pad(x, (L, R, U, D))
    src = x.permute(1, 2, 0).contiguous() if hwc else x
    n = ref.numel()
    out = torch.full((n + 8,), 7.0, device=DEV, dtype=TDT[dt])
    a = pkg.PadArgs()
    a.source, a.dest, a.C, a.H, a.W = src.data_ptr(), out.data_ptr(), C, H, W
    a.T_LPAD, a.T_RPAD, a.T_UPAD, a.T_DPAD, a.HWC_lay = L, R, U, D, hwc
    pkg.call("pad_tensor" if dt == "fp32" else "pad_tensor_fp16", a)
    sync(gpu)
    want = ref.permute(1, 2, 0).contiguous() if hwc else ref
    assert same_bits(out[:n], want.reshape(-1))
    assert bool((out[n:] == 7.0).all())
