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


def test_layers_in_a_row_with_the_copy_handed_on_replay_as_a_hip_graph(pkg, gpu):
    """Two 3x3 layers with the blocked copy handed from the first layer's forward kernel to the second layer's forward
    and weight-gradient calls (ptl_conv2d_fp16_cache_prepare, _fw_batched_chained, _wg_batched_cached), captured once
    on a stream of the caller's: every replay, with the outputs and the copy overwritten in between, reproduces the
    eager result bit for bit."""
    Ci, H, Cm, Co, ns = 64, 14, 128, 64, 12
    pad = (1, 1, 1, 1)
    g = torch.Generator(device="cpu").manual_seed(11)
    x = (torch.rand(ns, Ci, H, H, generator=g) - 0.5).half().to(DEV)
    w1 = ((torch.rand(Cm, Ci, 3, 3, generator=g) - 0.5) * 0.2).half().to(DEV)
    w2 = ((torch.rand(Co, Cm, 3, 3, generator=g) - 0.5) * 0.2).half().to(DEV)
    dy2 = (torch.rand(ns, Co, H, H, generator=g) - 0.5).half().to(DEV)
    y1 = torch.zeros(ns, Cm, H, H, device=DEV).half()
    y2, dw2 = torch.zeros_like(dy2), torch.zeros_like(w2)
    a1, k1 = hp.conv2d_args(pkg, x, None, w1, None, y1, None, Ci, H, H, Cm, 3, 3, H, H, pad, (1, 1))
    a2, k2 = hp.conv2d_args(pkg, y1, None, w2, dw2, y2, dy2, Cm, H, H, Co, 3, 3, H, H, pad, (1, 1))
    nbytes = gpu.ptl_conv2d_fp16_cache_bytes(ctypes.byref(a2), ns)
    assert nbytes > 0
    buf = torch.full((nbytes,), 0x3c, dtype=torch.uint8, device=DEV)
    c = pkg.ConvCache()
    c.buf, c.bytes = buf.data_ptr(), nbytes

    def step():
        assert gpu.ptl_conv2d_fp16_cache_prepare(ctypes.byref(a2), ns, ctypes.byref(c)) == 0
        assert gpu.ptl_conv2d_fp16_fw_batched_chained(ctypes.byref(a1), ns, None, ctypes.byref(c)) == 0
        assert c.valid == 1
        assert gpu.ptl_conv2d_fp16_fw_batched_chained(ctypes.byref(a2), ns, ctypes.byref(c), None) == 0
        assert gpu.ptl_conv2d_fp16_wg_batched_cached(ctypes.byref(a2), ns, ctypes.byref(c)) == 0

    side = torch.cuda.Stream()
    gpu.ptl_set_gemm_path(5)
    gpu.ptl_set_stream(ctypes.c_void_p(side.cuda_stream))
    try:
        with torch.cuda.stream(side):
            step()  # (eager: the result to reproduce, and the library's buffers at their size)
            side.synchronize()
        eager = [t.clone() for t in (y1, y2, dw2)]
        ref = torch.nn.functional.conv2d(torch.nn.functional.conv2d(x.double(), w1.double(), padding=1).half().double(),
                                         w2.double(), padding=1)
        assert float((eager[1].double() - ref).norm() / ref.norm()) <= 2e-3
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
        for k in range(3):
            for t in (y1, y2, dw2):
                t.fill_(float(k + 2))
            buf.fill_(0x3c + k)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for t, e in zip((y1, y2, dw2), eager):
                assert torch.equal(t, e)
    finally:
        gpu.ptl_set_gemm_path(0)
        gpu.ptl_set_stream(None)
        assert gpu.ptl_sync() == 0
