"""GPU parity of the fp32 attention step against the CPU oracle, through the C ABI.

Bar: relative L2 error <= 1e-4 for every tensor the step produces (fp32).  The backward pass is fed the
ORACLE's forward results, so a forward deviation cannot hide in it.
"""
import ctypes

import numpy as np
import pytest
import torch

import helpers as hp

pytestmark = pytest.mark.gpu

TOL = 1e-4
FW_OUT = ("q", "k", "v", "p", "att", "y")
BW_OUT = ("wo", "att", "p", "q", "k", "v", "wq", "wk", "wv", "x")


def oracle_step(pkg, orc, d, dy, x0, ns, L, E, F, heads):
    lib = orc.load()
    sh = hp.mhsa_shapes(ns, L, E, F, heads)
    data = dict(d)
    for n in FW_OUT:
        data[n] = np.zeros(sh[n], np.float32)
    diff = {n: np.zeros(sh[n], np.float32) for n in ("q", "k", "v", "att", "p", "wo")}
    for n in ("wq", "wk", "wv"):
        diff[n] = np.zeros((F, E), np.float32)
    diff["x"] = x0.copy()
    diff["y"] = dy
    a, keep = hp.mhsa_args(pkg, data, diff, L, E, F, heads)
    lib.orc_mhsa_fw_fp32(ctypes.byref(a), ns)
    lib.orc_mhsa_bw_fp32(ctypes.byref(a), ns)
    return data, diff


def gpu_step(pkg, gpu, d, dy, x0, fw_ref, ns, L, E, F, heads, device, named):
    """Forward from the inputs, backward from the oracle's forward state.  Returns (forward data, gradients)."""
    sh = hp.mhsa_shapes(ns, L, E, F, heads)
    mk = (lambda z: torch.from_numpy(np.ascontiguousarray(z)).cuda()) if device else (lambda z: np.ascontiguousarray(z).copy())
    zeros = lambda s: mk(np.full(s, 7.0, np.float32))  # outputs start dirty: they must be overwritten
    data = {n: mk(v) for n, v in d.items()}
    for n in FW_OUT:
        data[n] = zeros(sh[n])
    a, keep = hp.mhsa_args(pkg, data, {}, L, E, F, heads)
    if named:
        assert ns == 1
        gpu.pulp_mhsa_fp32_fw_cl(ctypes.byref(a))
        assert gpu.ptl_last_status() == 0, gpu.ptl_last_error().decode()
    else:
        assert gpu.ptl_mhsa_fp32_fw_batched(ctypes.byref(a), ns) == 0, gpu.ptl_last_error().decode()
    data2 = {n: mk(v) for n, v in d.items()}
    for n in FW_OUT:
        data2[n] = mk(fw_ref[n])
    diff = {n: zeros(sh[n]) for n in ("q", "k", "v", "att", "p", "wo")}
    for n in ("wq", "wk", "wv"):
        diff[n] = zeros((F, E))
    diff["x"] = mk(x0)
    diff["y"] = mk(dy)
    b, keep2 = hp.mhsa_args(pkg, data2, diff, L, E, F, heads)
    if named:
        gpu.pulp_mhsa_fp32_bw_cl(ctypes.byref(b))
        assert gpu.ptl_last_status() == 0, gpu.ptl_last_error().decode()
    else:
        assert gpu.ptl_mhsa_fp32_bw_batched(ctypes.byref(b), ns) == 0, gpu.ptl_last_error().decode()
    if device:
        assert gpu.ptl_sync() == 0
        back = lambda z: z.cpu().numpy()
    else:
        back = lambda z: z
    return {n: back(data[n]) for n in FW_OUT}, {n: back(diff[n]) for n in BW_OUT}


# (ns, L, E, F, heads): tiny reference default (tests/test_mhsa_fp32/Makefile: L=E=10, F=160, 5 heads),
# ragged sizes, one head, head sizes 16/32/64/128, and the ViT-Tiny geometry L=197 E=192 3 x 64.
CASES = [
    (1, 10, 10, 160, 5),
    (3, 7, 12, 8, 2),
    (2, 33, 16, 24, 3),
    (1, 65, 24, 64, 1),
    (2, 100, 40, 256, 2),
    (1, 197, 192, 192, 3),
    (3, 197, 192, 192, 3),
]


# every case with device pointers; with host pointers (staged by the library) all but the largest
@pytest.mark.parametrize("case,device", [(c, True) for c in CASES] + [(c, False) for c in CASES if c[0] * c[1] <= 300])
def test_mhsa_step_matches_oracle(pkg, orc, gpu, case, device):
    ns, L, E, F, heads = case
    seed = 0xC0DE0004 + 97 * L + ns
    d, dy = hp.mhsa_inputs(seed, ns, L, E, F, heads)
    x0 = hp.uniform(seed + 31, (ns, E, L))
    ref_data, ref_diff = oracle_step(pkg, orc, d, dy, x0, ns, L, E, F, heads)
    got_data, got_diff = gpu_step(pkg, gpu, d, dy, x0, ref_data, ns, L, E, F, heads, device, named=False)
    for n in FW_OUT:
        assert hp.rel_l2(got_data[n], ref_data[n]) <= TOL, "forward %s" % n
    for n in BW_OUT:
        assert hp.rel_l2(got_diff[n], ref_diff[n]) <= TOL, "backward %s" % n


def test_mhsa_reference_named_entry_points(pkg, orc, gpu):
    ns, L, E, F, heads = 1, 10, 10, 160, 5
    d, dy = hp.mhsa_inputs(0xC0DE0044, ns, L, E, F, heads)
    x0 = np.zeros((ns, E, L), np.float32)
    ref_data, ref_diff = oracle_step(pkg, orc, d, dy, x0, ns, L, E, F, heads)
    got_data, got_diff = gpu_step(pkg, gpu, d, dy, x0, ref_data, ns, L, E, F, heads, False, named=True)
    for n in FW_OUT:
        assert hp.rel_l2(got_data[n], ref_data[n]) <= TOL, "forward %s" % n
    for n in BW_OUT:
        assert hp.rel_l2(got_diff[n], ref_diff[n]) <= TOL, "backward %s" % n


def test_mhsa_batch_is_per_sample(pkg, orc, gpu):
    """A batch equals its samples run one by one: activations per sample, weight gradients summed."""
    ns, L, E, F, heads = 4, 50, 32, 64, 2
    d, dy = hp.mhsa_inputs(0xC0DE0045, ns, L, E, F, heads)
    x0 = np.zeros((ns, E, L), np.float32)
    ref_data, _ = oracle_step(pkg, orc, d, dy, x0, ns, L, E, F, heads)
    full_d, full_g = gpu_step(pkg, gpu, d, dy, x0, ref_data, ns, L, E, F, heads, True, named=False)
    acc = {n: 0.0 for n in ("wo", "wq", "wk", "wv")}
    for b in range(ns):
        db = dict(d)
        db["x"] = d["x"][b:b + 1]
        rd = {n: ref_data[n][b:b + 1] for n in FW_OUT}
        one_d, one_g = gpu_step(pkg, gpu, db, dy[b:b + 1], x0[b:b + 1], rd, 1, L, E, F, heads, True, named=False)
        for n in FW_OUT:
            assert np.array_equal(one_d[n][0], full_d[n][b]), n
        for n in ("att", "p", "q", "k", "v", "x"):
            assert np.array_equal(one_g[n][0], full_g[n][b]), n
        for n in acc:
            acc[n] = acc[n] + one_g[n].astype(np.float64)
    for n in acc:
        assert hp.rel_l2(full_g[n], acc[n]) <= 1e-5, n


def test_softmax_entry_points(pkg, orc, gpu):
    H, W = 37, 197
    x = hp.normal(0x50F70001, (H, W), 3.0)
    g = hp.uniform(0x50F70002, (H, W))
    ref = {n: np.zeros((H, W), np.float32) for n in ("out", "gi")}
    rmx, rsm = np.zeros(H, np.float32), np.zeros(H, np.float32)
    a = pkg.SoftmaxArgs()
    a.input_data, a.output_data, a.maxes, a.sums, a.H, a.W = (pkg.addr(x), pkg.addr(ref["out"]), pkg.addr(rmx),
                                                              pkg.addr(rsm), H, W)
    orc.load().orc_softmax_fw_fp32(ctypes.byref(a))
    b = pkg.SoftmaxArgs()
    b.input_diff, b.output_data, b.output_diff, b.H, b.W = pkg.addr(ref["gi"]), pkg.addr(ref["out"]), pkg.addr(g), H, W
    orc.load().orc_softmax_bw_fp32(ctypes.byref(b))
    out, gi = np.full((H, W), 7.0, np.float32), np.full((H, W), 7.0, np.float32)
    mx, sm = np.zeros(H, np.float32), np.zeros(H, np.float32)
    a.output_data, a.maxes, a.sums = pkg.addr(out), pkg.addr(mx), pkg.addr(sm)
    gpu.pulp_softmax_fp32_fw_cl(ctypes.byref(a))
    assert gpu.ptl_last_status() == 0, gpu.ptl_last_error().decode()
    assert hp.rel_l2(out, ref["out"]) <= 1e-5
    assert np.array_equal(mx, rmx)
    assert hp.rel_l2(sm, rsm) <= 1e-5
    b.input_diff = pkg.addr(gi)
    gpu.pulp_softmax_fp32_bw_cl(ctypes.byref(b))
    assert gpu.ptl_last_status() == 0, gpu.ptl_last_error().decode()
    assert hp.rel_l2(gi, ref["gi"]) <= 1e-5
    # in place, as the forward may be called
    y = x.copy()
    a.input_data = a.output_data = pkg.addr(y)
    gpu.pulp_softmax_fp32_fw_cl(ctypes.byref(a))
    assert gpu.ptl_last_status() == 0
    assert np.array_equal(y, out)


def test_mhsa_rejects_bad_geometry(pkg, gpu):
    ns, L, E, F, heads = 1, 8, 8, 10, 3  # F not divisible by heads
    sh = hp.mhsa_shapes(ns, L, E, F, heads)
    data = {n: np.zeros(sh[n], np.float32) for n in hp.MHSA_TENSORS}
    a, keep = hp.mhsa_args(pkg, data, {}, L, E, F, heads)
    assert gpu.ptl_mhsa_fp32_fw_batched(ctypes.byref(a), 1) == 1
    assert b"geometry" in gpu.ptl_last_error()
    assert np.all(data["y"] == 0)
