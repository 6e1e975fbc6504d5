"""Shared test helpers: seeded inputs, argument-struct builders, error metrics."""
import ctypes

import numpy as np

MASK = (1 << 64) - 1


def splitmix64(seed, n):
    """n 64-bit words of the SplitMix64 sequence started at `seed` (vectorised)."""
    idx = np.arange(1, n + 1, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = np.uint64(seed & MASK) + idx * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z


def uniform(seed, shape, lo=-1.0, hi=1.0, dtype=np.float32):
    n = int(np.prod(shape))
    u = (splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
    return (lo + (hi - lo) * u).reshape(shape).astype(dtype)


def normal(seed, shape, sigma=1.0, dtype=np.float32):
    n = int(np.prod(shape))
    u1 = ((splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / ((1 << 53) + 1))
    u2 = (splitmix64(seed ^ 0xABCDEF, n) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (sigma * z).reshape(shape).astype(dtype)


def rel_l2(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    den = np.linalg.norm(ref)
    return float(np.linalg.norm(got - ref) / (den if den > 0 else 1.0))


def np_dtype(dt):
    return np.float32 if dt == "fp32" else np.float16


def ptr(b):
    return ctypes.pointer(b)


class Keep(list):
    """Holds the objects an argument struct points to."""


def conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, Hk, Wk, Ho, Wo, pad=(0, 0, 0, 0), stride=(1, 1), hwc=0,
                im2col=1, bias=None, dbias=None, i2c=None, bt=None):
    """Conv2D_args over the given tensors; pad = (L, R, U, D), stride = (h, w)."""
    keep = Keep()
    bi = pkg.blob(x, dx, Ci, H, W)
    bw = pkg.blob(w, dw, Ci, Hk, Wk, dim=Co * Ci * Hk * Wk)
    bo = pkg.blob(y, dy, Co, Ho, Wo)
    bb = pkg.blob(bias, dbias, 1, 1, Co)
    keep += [bi, bw, bo, bb, x, dx, w, dw, y, dy, bias, dbias, i2c, bt]
    a = pkg.Conv2DArgs()
    a.input, a.coeff, a.output = ptr(bi), ptr(bw), ptr(bo)
    if bias is not None or dbias is not None:
        a.bias = ptr(bb)
        a.USE_BIASES = 1
    a.Lpad, a.Rpad, a.Upad, a.Dpad = pad
    a.stride_h, a.stride_w = stride
    a.i2c_buffer = pkg.addr(i2c)
    a.bt_buffer = pkg.addr(bt)
    a.HWC = hwc
    a.USE_IM2COL = im2col
    return a, keep


def pw_args(pkg, x, dx, w, dw, y, dy, Ci, Co, H, W, hwc=0):
    keep = Keep()
    bi = pkg.blob(x, dx, Ci, H, W)
    bw = pkg.blob(w, dw, Ci, 1, 1, dim=Co * Ci)
    bo = pkg.blob(y, dy, Co, H, W)
    keep += [bi, bw, bo, x, dx, w, dw, y, dy]
    a = pkg.PointWiseConvArgs()
    a.input, a.coeff, a.output = ptr(bi), ptr(bw), ptr(bo)
    a.HWC = hwc
    return a, keep


def dw_args(pkg, dt, x, dx, w, dw, y, dy, C, H, W, Hk, Wk, Ho, Wo, pad=(0, 0, 0, 0), stride=(1, 1)):
    keep = Keep()
    bi = pkg.blob(x, dx, C, H, W)
    bw = pkg.blob(w, dw, 1, Hk, Wk, dim=C * Hk * Wk)
    bo = pkg.blob(y, dy, C, Ho, Wo)
    keep += [bi, bw, bo, x, dx, w, dw, y, dy]
    if dt == "fp32":
        a = pkg.DepthWiseConvArgs()
        a.stride_h, a.stride_w = stride
    else:
        assert tuple(stride) == (1, 1)
        a = pkg.DepthWiseConvArgsFp16()
    a.input, a.coeff, a.output = ptr(bi), ptr(bw), ptr(bo)
    a.Lpad, a.Rpad, a.Upad, a.Dpad = pad
    return a, keep


def linear_args(pkg, x, dx, w, dw, y, dy, n_in, n_out, bias=None, dbias=None):
    keep = Keep()
    bi = pkg.blob(x, dx, 1, 1, n_in, dim=n_in)
    bw = pkg.blob(w, dw, 1, n_out, n_in, dim=n_in * n_out)
    bo = pkg.blob(y, dy, 1, 1, n_out, dim=n_out)
    bb = pkg.blob(bias, dbias, 1, 1, n_out)
    keep += [bi, bw, bo, bb, x, dx, w, dw, y, dy, bias, dbias]
    a = pkg.LinearArgs()
    a.input, a.coeff, a.output = ptr(bi), ptr(bw), ptr(bo)
    if bias is not None or dbias is not None:
        a.bias = ptr(bb)
        a.use_biases = 1
    return a, keep


def mm_args(pkg, A, B, Cm, N, M, K, trans_B):
    a = pkg.MatMulArgs()
    a.A, a.B, a.C = pkg.addr(A), pkg.addr(B), pkg.addr(Cm)
    a.N, a.M, a.K, a.trans_B = N, M, K, trans_B
    return a


def conv_out(n, k, p0, p1, s):
    return (n - k + p0 + p1) // s + 1


MHSA_TENSORS = ("x", "wq", "wk", "wv", "bq", "bk", "bv", "wo", "q", "k", "v", "att", "p", "y")


def mhsa_shapes(ns, L, E, F, heads):
    """Shapes of the attention tensors (data and diff alike; weight gradients of wq/wk/wv are F x E)."""
    return {"x": (ns, E, L), "wq": (E, F), "wk": (E, F), "wv": (E, F), "bq": (F,), "bk": (F,), "bv": (F,),
            "wo": (E, F), "q": (ns, F, L), "k": (ns, F, L), "v": (ns, F, L), "att": (ns, F, L),
            "p": (ns, heads, L, L), "y": (ns, E, L)}


def mhsa_args(pkg, data, diff, L, E, F, heads):
    """Mhsa_args over dicts of tensors keyed like MHSA_TENSORS (missing entries -> NULL), blob geometry as in
    tests/test_mhsa_fp32/net.c of the reference (input H = L, W = E; attention_map W = F)."""
    keep = Keep()
    geo = {"x": (1, L, E), "wq": (1, F, E), "wk": (1, F, E), "wv": (1, F, E), "bq": (1, 1, F), "bk": (1, 1, F),
           "bv": (1, 1, F), "wo": (1, E, F), "q": (1, L, F), "k": (1, L, F), "v": (1, L, F), "att": (1, L, F),
           "p": (1, heads, L * L), "y": (1, L, E)}
    blobs = {}
    for n in MHSA_TENSORS:
        c, h, w = geo[n]
        blobs[n] = pkg.blob(data.get(n), diff.get(n), c, h, w)
        keep += [blobs[n], data.get(n), diff.get(n)]
    a = pkg.MhsaArgs()
    a.input, a.output = ptr(blobs["x"]), ptr(blobs["y"])
    a.n_heads = heads
    a.coeff_in_q, a.coeff_in_k, a.coeff_in_v = ptr(blobs["wq"]), ptr(blobs["wk"]), ptr(blobs["wv"])
    a.bias_in_q, a.bias_in_k, a.bias_in_v = ptr(blobs["bq"]), ptr(blobs["bk"]), ptr(blobs["bv"])
    a.coeff_out = ptr(blobs["wo"])
    a.q, a.k, a.v = ptr(blobs["q"]), ptr(blobs["k"]), ptr(blobs["v"])
    a.attention_map, a.softmax_buffer = ptr(blobs["att"]), ptr(blobs["p"])
    return a, keep


def mhsa_inputs(seed, ns, L, E, F, heads):
    """Seeded inputs: tokens N(0,1), Xavier-uniform weights, small biases, output gradient U[-1,1]."""
    sh = mhsa_shapes(ns, L, E, F, heads)
    lim = float(np.sqrt(6.0 / (E + F)))
    d = {"x": normal(seed, sh["x"])}
    for i, n in enumerate(("wq", "wk", "wv", "wo")):
        d[n] = uniform(seed + 1 + i, sh[n], -lim, lim)
    for i, n in enumerate(("bq", "bk", "bv")):
        d[n] = uniform(seed + 11 + i, sh[n], -0.1, 0.1)
    dy = uniform(seed + 21, sh["y"])
    return d, dy


def act_args(pkg, x, dx, y, dy, dim):
    keep = Keep()
    bi, bo = pkg.blob(x, dx, 1, 1, dim, dim=dim), pkg.blob(y, dy, 1, 1, dim, dim=dim)
    keep += [bi, bo, x, dx, y, dy]
    a = pkg.ActArgs()
    a.input, a.output = ptr(bi), ptr(bo)
    return a, keep


def skip_args(pkg, skip, dskip, lout, dlout, out, dout, dim, skip_in_grad=0):
    keep = Keep()
    bs, bl, bo = (pkg.blob(skip, dskip, 1, 1, dim, dim=dim), pkg.blob(lout, dlout, 1, 1, dim, dim=dim),
                  pkg.blob(out, dout, 1, 1, dim, dim=dim))
    keep += [bs, bl, bo, skip, dskip, lout, dlout, out, dout]
    a = pkg.SkipConnArgs()
    a.skip, a.lout, a.output = ptr(bs), ptr(bl), ptr(bo)
    a.skip_in_grad = skip_in_grad
    return a, keep


def pool_args(pkg, x, dx, y, dy, C, H, W, Ho, Wo, Hk, Wk, Hs, Ws):
    keep = Keep()
    bi, bo = pkg.blob(x, dx, C, H, W), pkg.blob(y, dy, C, Ho, Wo)
    keep += [bi, bo, x, dx, y, dy]
    a = pkg.PoolArgs()
    a.input, a.output = ptr(bi), ptr(bo)
    a.Hker, a.Wker, a.Hstride, a.Wstride = Hk, Wk, Hs, Ws
    return a, keep


def loss_args(pkg, logits, dlogits, target, loss, ncls):
    keep = Keep()
    bo = pkg.blob(logits, dlogits, 1, 1, ncls, dim=ncls)
    keep += [bo, logits, dlogits, target, loss]
    a = pkg.LossArgs()
    a.output = ptr(bo)
    a.target, a.wr_loss = pkg.addr(target), pkg.addr(loss)
    return a, keep


def optim_args(pkg, dt, w, dw, b, db, lr, lam):
    keep = Keep()
    bw = pkg.blob(w, dw, 1, 1, int(np.prod(w.shape)), dim=int(np.prod(w.shape)))
    keep += [bw, w, dw, b, db]
    a = pkg.OptimArgs() if dt == "fp32" else pkg.OptimArgsFp16()
    a.weights = ptr(bw)
    if b is not None:
        bb = pkg.blob(b, db, 1, 1, int(np.prod(b.shape)), dim=int(np.prod(b.shape)))
        keep.append(bb)
        a.biases = ptr(bb)
        a.use_biases = 1
    if dt == "fp32":
        a.learning_rate, a.weight_decay_lambda = lr, lam
    else:
        a.learning_rate = int(np.float16(lr).view(np.uint16))
        a.weight_decay_lambda = int(np.float16(lam).view(np.uint16))
    return a, keep


def batch_norm_args(pkg, x, y, w, b, eps, B, C, H, W, dx=None, dy=None, dw=None, db=None):
    keep = Keep()
    bi, bo = pkg.blob(x, dx, C, H, W), pkg.blob(y, dy, C, H, W)
    bw, bb = pkg.blob(w, dw, C, 1, 1, dim=C), pkg.blob(b, db, C, 1, 1, dim=C)
    keep += [bi, bo, bw, bb, x, y, w, b, eps, dx, dy, dw, db]
    a = pkg.BatchNormArgs()
    a.input, a.output = ptr(bi), ptr(bo)
    a.coeff, a.bias = ptr(bw), ptr(bb)
    a.weight_data, a.bias_data, a.eps = pkg.addr(w), pkg.addr(b), pkg.addr(eps)
    a.B, a.C, a.H, a.W = B, C, H, W
    a.batch_size = B
    return a, keep
