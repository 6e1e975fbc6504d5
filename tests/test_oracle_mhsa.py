"""Pins of the attention oracle (CPU only): every check compares against something the oracle did not compute.

* approximate exponential: bit-exact against an integer evaluation of its definition, and within the method's
  error band of exp();
* q_rsqrt: one Newton step from the magic constant, within 0.2 % of 1/sqrt;
* forward: a float64 torch model of the reference's golden network (linear projections with bias, per-head
  scaled dot products, softmax, value mix, output projection) in which only the exponential is the float32
  approximation;
* softmax backward: autograd of the exact softmax taken at log(P) (whose Jacobian is diag(P) - P P^T);
* backward: autograd through the float64 model with that softmax Jacobian.
"""
import ctypes

import numpy as np
import pytest
import torch

import helpers as hp


def fastexp_np(x):
    """fastexp_gist of the reference's golden model (tests/test_mhsa_fp32/utils/SoftmaxFastExp.py), in numpy."""
    x = np.asarray(x, dtype=np.float32)
    y = x * np.float32(12102203.17133801) + np.float32(1064986823.010288)
    y = np.where(y < np.float32(8388608), np.float32(0), y)
    y = np.where(y > np.float32(2139095040), np.float32(2139095040), y).astype(np.float32)
    return y.astype(np.uint32).view(np.float32)


def rsqrt_np(x):
    y = np.asarray((x,), dtype=np.float32)
    i = np.int32(0x5F3759DF) - (y.view(np.int32) >> 1)
    z = i.view(np.float32)
    return float((z * (np.float32(1.5) - (y * np.float32(0.5) * z * z)))[0])


def test_fastexp_and_rsqrt(orc):
    lib = orc.load()
    xs = np.concatenate([np.linspace(-100, 0, 4001), [-87.4, -87.3, -1e-8, 0.0, 1.0, 88.0, 89.5]]).astype(np.float32)
    got = np.array([lib.orc_fastexp_gist(float(x)) for x in xs], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32), fastexp_np(xs).view(np.uint32))
    inside = (xs > -80) & (xs <= 0)
    rel = np.abs(got[inside] / np.exp(xs[inside].astype(np.float64)) - 1)
    assert rel.max() < 0.07  # Schraudolph's construction: a few percent
    for h in (1.0, 8.0, 32.0, 64.0, 100.0):
        r = lib.orc_q_rsqrt(h)
        assert r == rsqrt_np(h)
        assert abs(r * np.sqrt(h) - 1) < 2e-3


class SoftmaxApprox(torch.autograd.Function):
    """Forward: approximate-exponential softmax in float32; backward: the exact softmax Jacobian at the output."""

    @staticmethod
    def forward(ctx, s):
        s32 = s.detach().numpy().astype(np.float32)
        e = fastexp_np(s32 - s32.max(-1, keepdims=True))
        p = torch.from_numpy((e / e.sum(-1, keepdims=True, dtype=np.float32)).astype(np.float64))
        ctx.save_for_backward(p)
        return p

    @staticmethod
    def backward(ctx, g):
        (p,) = ctx.saved_tensors
        logp = torch.log(p.clamp_min(1e-300)).requires_grad_(True)
        with torch.enable_grad():
            out = torch.softmax(logp, -1) * p.sum(-1, keepdim=True)
            (gi,) = torch.autograd.grad(out, logp, g)
        return gi


def torch_model(d, heads, scale):
    """Golden network in float64: x is (ns, E, L) with tokens as columns; weights as the oracle stores them."""
    x = d["x"].transpose(1, 2)  # (ns, L, E)
    q = x @ d["wq"] + d["bq"]  # (ns, L, F)
    k = x @ d["wk"] + d["bk"]
    v = x @ d["wv"] + d["bv"]
    ns, L, F = q.shape
    H = F // heads
    sp = lambda t: t.reshape(ns, L, heads, H).permute(0, 2, 1, 3)  # (ns, heads, L, H)
    s = (sp(q) @ sp(k).transpose(-1, -2)) * scale
    p = SoftmaxApprox.apply(s)
    att = (p @ sp(v)).permute(0, 2, 1, 3).reshape(ns, L, F)
    y = att @ d["wo"].transpose(0, 1)  # (ns, L, E)
    return q, k, v, p, att, y


CASES = [(1, 10, 10, 20, 5), (2, 7, 12, 8, 2), (1, 33, 16, 24, 3), (2, 40, 24, 64, 1)]


@pytest.mark.parametrize("case", CASES)
def test_mhsa_oracle_against_float64_model(pkg, orc, case):
    ns, L, E, F, heads = case
    lib = orc.load()
    d, dy = hp.mhsa_inputs(0xA77E0000 + L, ns, L, E, F, heads)
    sh = hp.mhsa_shapes(ns, L, E, F, heads)
    data = dict(d)
    for n in ("q", "k", "v", "att", "p", "y"):
        data[n] = np.zeros(sh[n], np.float32)
    diff = {n: np.zeros(sh[n], np.float32) for n in ("x", "q", "k", "v", "att", "p", "wo")}
    for n in ("wq", "wk", "wv"):
        diff[n] = np.zeros((F, E), np.float32)
    diff["y"] = dy
    x0 = hp.uniform(0xA77E9999, sh["x"])  # the input gradient is added to what the buffer holds
    diff["x"][...] = x0
    a, keep = hp.mhsa_args(pkg, data, diff, L, E, F, heads)
    lib.orc_mhsa_fw_fp32(ctypes.byref(a), ns)
    lib.orc_mhsa_bw_fp32(ctypes.byref(a), ns)

    t = {n: torch.tensor(v.astype(np.float64), requires_grad=n in ("x", "wq", "wk", "wv", "wo")) for n, v in d.items()}
    scale = rsqrt_np(float(F // heads))
    q, k, v, p, att, y = torch_model(t, heads, scale)
    tr = lambda z: z.detach().transpose(1, 2).numpy()
    assert hp.rel_l2(data["q"], tr(q)) < 2e-6
    assert hp.rel_l2(data["k"], tr(k)) < 2e-6
    assert hp.rel_l2(data["v"], tr(v)) < 2e-6
    assert hp.rel_l2(data["p"], p.detach().numpy()) < 2e-5
    assert hp.rel_l2(data["att"], tr(att)) < 2e-5
    assert hp.rel_l2(data["y"], tr(y)) < 2e-5
    for tt in (q, k, v, p, att):
        tt.retain_grad()
    y.backward(torch.tensor(dy.astype(np.float64)).transpose(1, 2))
    assert hp.rel_l2(diff["wo"], t["wo"].grad.numpy()) < 5e-5
    assert hp.rel_l2(diff["att"], tr(att.grad)) < 5e-5
    assert hp.rel_l2(diff["v"], tr(v.grad)) < 5e-5
    assert hp.rel_l2(diff["p"], p.grad.numpy()) < 5e-5
    assert hp.rel_l2(diff["q"], tr(q.grad)) < 5e-5
    assert hp.rel_l2(diff["k"], tr(k.grad)) < 5e-5
    for n in ("wq", "wk", "wv"):  # gradients come out F x E, the weights are stored E x F
        assert hp.rel_l2(diff[n], t[n].grad.numpy().T) < 5e-5
    assert hp.rel_l2(diff["x"] - x0, t["x"].grad.numpy()) < 5e-5


def test_softmax_rows(pkg, orc):
    lib = orc.load()
    H, W = 9, 37
    x = hp.normal(0x50F7, (H, W), 3.0)
    out, mx, sm = np.zeros((H, W), np.float32), np.zeros(H, np.float32), np.zeros(H, np.float32)
    a = pkg.SoftmaxArgs()
    a.input_data, a.output_data, a.maxes, a.sums, a.H, a.W = pkg.addr(x), pkg.addr(out), pkg.addr(mx), pkg.addr(sm), H, W
    lib.orc_softmax_fw_fp32(ctypes.byref(a))
    e = fastexp_np(x - x.max(-1, keepdims=True)).astype(np.float64)
    assert hp.rel_l2(out, e / e.sum(-1, keepdims=True)) < 1e-6
    assert np.array_equal(mx, x.max(-1))
    assert np.abs(out.sum(-1) - 1).max() < 1e-5
    exact = torch.softmax(torch.tensor(x.astype(np.float64)), -1).numpy()
    assert np.abs(out - exact).max() < 0.05  # the approximation, not the arithmetic
    # backward against autograd of the exact softmax at log(out)
    g = hp.uniform(0x50F8, (H, W))
    gi = np.zeros((H, W), np.float32)
    b = pkg.SoftmaxArgs()
    b.input_diff, b.output_data, b.output_diff, b.sums, b.H, b.W = (pkg.addr(gi), pkg.addr(out), pkg.addr(g),
                                                                    pkg.addr(sm), H, W)
    lib.orc_softmax_bw_fp32(ctypes.byref(b))
    lp = torch.log(torch.tensor(out.astype(np.float64))).requires_grad_(True)
    o = torch.softmax(lp, -1) * torch.tensor(out.astype(np.float64)).sum(-1, keepdim=True)
    (ref,) = torch.autograd.grad(o, lp, torch.tensor(g.astype(np.float64)))
    assert hp.rel_l2(gi, ref.numpy()) < 1e-5
