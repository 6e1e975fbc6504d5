"""The library's own device buffers and its stream under HIP graph capture: ptl_reserve / ptl_reserved, the refusal
to grow a buffer or to leave a stream while that stream is being captured (the capture stays valid), and the same
call captured and replayed once the buffer is there."""
import ctypes

import numpy as np
import pytest
import torch

import helpers as hp

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def reserved(lib):
    ws, sc = ctypes.c_size_t(0), ctypes.c_size_t(0)
    lib.ptl_reserved(ctypes.byref(ws), ctypes.byref(sc))
    return ws.value, sc.value


def test_reserve_grows_and_reports(pkg, gpu):
    ws0, sc0 = reserved(gpu)
    assert gpu.ptl_reserve(ws0 + (3 << 20), 0) == 0, gpu.ptl_last_error().decode()
    ws1, sc1 = reserved(gpu)
    assert ws1 >= ws0 + (3 << 20) and sc1 == sc0
    assert gpu.ptl_reserve(1, 1) == 0  # never shrinks
    ws2, sc2 = reserved(gpu)
    assert ws2 == ws1 and sc2 >= max(sc1, 1)


def test_growth_and_stream_switch_are_refused_under_capture_and_reserve_makes_the_call_capturable(pkg, gpu):
    """A strided input gradient on the general GEMM route zero-stuffs the output gradient into the library's scratch
    buffer.  Captured when that buffer is too small, the call fails with status 2 and names ptl_reserve; the capture
    survives; after ptl_reserve the same call is captured, and its replays reproduce the eager result bit for bit."""
    _, sc0 = reserved(gpu)
    if sc0 > (256 << 20):
        pytest.skip("the scratch buffer has already grown beyond what this test can outgrow cheaply")
    Ci, Co, H, K, s = 4, 8, 127, 3, 2
    Ho = hp.conv_out(H, K, 1, 1, s)
    Hd = (Ho - 1) * s + 1
    per_sample = Co * Hd * Hd * 4
    ns = (sc0 + (1 << 20)) // per_sample + 2
    need = ns * per_sample
    assert need > sc0
    g = torch.Generator(device="cpu").manual_seed(5)
    w = (torch.rand(Co, Ci, K, K, generator=g) - 0.5).to(DEV)
    dy = (torch.rand(ns, Co, Ho, Ho, generator=g) - 0.5).to(DEV)
    dx = torch.zeros(ns, Ci, H, H, device=DEV)
    a, keep = hp.conv2d_args(pkg, None, dx, w, None, None, dy, Ci, H, H, Co, K, K, Ho, Ho, (1, 1, 1, 1), (s, s))
    side = torch.cuda.Stream()
    gpu.ptl_set_gemm_path(1)
    gpu.ptl_set_stream(ctypes.c_void_p(side.cuda_stream))
    try:
        assert gpu.ptl_last_status() == 0
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            rc = gpu.ptl_conv2d_fp32_ig_batched(ctypes.byref(a), ns)
            msg = gpu.ptl_last_error().decode()
            gpu.ptl_set_stream(None)  # refused: the stream being left is capturing
            st_switch = gpu.ptl_last_status()
            assert gpu.ptl_copy_bytes(ctypes.c_void_p(w.data_ptr()), ctypes.c_void_p(dx.data_ptr()), 64) == 0
        assert rc == 2 and "ptl_reserve" in msg, (rc, msg)
        assert st_switch == 1
        assert reserved(gpu)[1] == sc0
        graph.replay()  # the capture was not invalidated: it holds the one copy
        torch.cuda.synchronize()
        assert torch.equal(dx.flatten()[:16], w.flatten()[:16])
        del graph
        # with the buffer reserved the call is captured ...
        assert gpu.ptl_reserve(0, need) == 0, gpu.ptl_last_error().decode()
        assert reserved(gpu)[1] >= need
        with torch.cuda.stream(side):
            assert gpu.ptl_conv2d_fp32_ig_batched(ctypes.byref(a), ns) == 0, gpu.ptl_last_error().decode()
            side.synchronize()
        eager = dx.clone()
        ref = torch.nn.grad.conv2d_input((ns, Ci, H, H), w.double(), dy.double(), stride=s, padding=1)
        assert float((eager.double() - ref).norm() / ref.norm()) <= 1e-4
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            rc = gpu.ptl_conv2d_fp32_ig_batched(ctypes.byref(a), ns)
        assert rc == 0, gpu.ptl_last_error().decode()
        # ... and every replay, with eager work between them, gives the eager result
        for _ in range(3):
            dx.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(dx, eager)
    finally:
        gpu.ptl_set_gemm_path(0)
        gpu.ptl_set_stream(None)
        assert gpu.ptl_sync() == 0
