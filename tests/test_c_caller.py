"""A compiled C caller: tests/c_caller/net.c (a reference-style net.c) is built with clang against include/ and
linked with libptl_hip.so, nothing else.  Without a GPU it must fail loudly ("no CPU fallback"); on the GPU its
results are checked against the CPU oracle run on the inputs the program wrote."""
import os
import subprocess

import numpy as np
import pytest

import helpers as hp

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLANG = "/opt/rocm/lib/llvm/bin/clang"
LIBDIR = os.path.join(ROOT, "pulp-trainlib_amd")


@pytest.fixture(scope="module")
def net_exe(tmp_path_factory, pkg):
    pkg.load()  # the library must be built
    exe = str(tmp_path_factory.mktemp("c_caller") / "net")
    subprocess.check_call([CLANG, "-std=gnu99", "-O1", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "c_caller", "net.c"), "-L", LIBDIR, "-lptl_hip",
                           "-Wl,-rpath," + LIBDIR, "-o", exe])
    return exe


def test_c_caller_fails_loudly_without_a_gpu(net_exe, tmp_path):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    res = subprocess.run([net_exe, "conv2d", str(tmp_path / "out.bin")], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                         text=True)
    assert res.returncode == 3
    assert "no CPU fallback" in res.stderr


def split(buf, shapes):
    out, pos = [], 0
    for s in shapes:
        n = int(np.prod(s))
        out.append(buf[pos:pos + n].reshape(s).copy())
        pos += n
    assert pos == buf.size
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("layer", ["conv2d", "linear", "pw", "dw"])
def test_c_caller_matches_oracle(net_exe, tmp_path, pkg, orc, gpu, layer):
    path = str(tmp_path / (layer + ".bin"))
    res = subprocess.run([net_exe, layer, path], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert res.returncode == 0, res.stderr
    buf = np.fromfile(path, dtype=np.float32)
    if layer == "conv2d":
        xs, ws, ys = (16, 32, 32), (32, 16, 3, 3), (32, 32, 32)
    elif layer == "linear":
        xs, ws, ys = (256,), (128, 256), (128,)
    elif layer == "pw":
        xs, ws, ys = (16, 100), (24, 16), (24, 100)
    else:
        xs, ws, ys = (8, 12, 12), (8, 3, 3), (8, 10, 10)
    x, w, dy, y, dw, dx = split(buf, (xs, ws, ys, ys, ws, xs))
    # the program's inputs are the SplitMix64 stream of the test helpers, seed 0xC0DE0001
    n = x.size + w.size + dy.size
    stream = hp.uniform(0xC0DE0001, (n,))
    assert np.array_equal(np.concatenate([x.ravel(), w.ravel(), dy.ravel()]), stream)
    ry, rdw, rdx = np.zeros_like(y), np.zeros_like(dw), np.zeros_like(dx)
    if layer == "conv2d":
        a, keep = hp.conv2d_args(pkg, x, rdx, w, rdw, ry, dy, 16, 32, 32, 32, 3, 3, 32, 32, (1, 1, 1, 1))
        name = "orc_conv2d_"
    elif layer == "linear":
        a, keep = hp.linear_args(pkg, x, rdx, w, rdw, ry, dy, 256, 128)
        name = "orc_linear_"
    elif layer == "pw":
        a, keep = hp.pw_args(pkg, x, rdx, w, rdw, ry, dy, 16, 24, 10, 10)
        name = "orc_conv_pw_"
    else:
        a, keep = hp.dw_args(pkg, "fp32", x, rdx, w, rdw, ry, dy, 8, 12, 12, 3, 3, 10, 10)
        name = "orc_conv_dw_"
    for s in ("fw", "wg", "ig"):
        orc.call(name + s, "fp32", a, 1)
    for what, got, ref in (("y", y, ry), ("dw", dw, rdw), ("dx", dx, rdx)):
        assert hp.rel_l2(got, ref) <= 1e-4, (layer, what)
