"""A ResNet-20-shaped (CIFAR geometry) training step assembled from the library's entry points, the way a
generated `net.c` of the reference strings its layer calls together: 3x3 stem, three stages of three residual
blocks (16/32/64 channels, stride-2 1x1 projection shortcuts), ReLU, global average pooling, a linear
classifier, cross-entropy and one gradient-descent update.  With `norm=True` every convolution is followed by
batch normalisation over the batch (the reference's forward, lib/sources/pulp_batchnorm_fp32.c:34, and this
library's backward for it).  Used by the GPU parity test and by the benchmark's detail table."""
import ctypes

import numpy as np

import helpers as hp


def resnet20_spec(num_classes=10):
    """[(name, cin, cout, k, stride)] of every convolution, in forward order, plus the block structure."""
    convs = [("stem", 3, 16, 3, 1)]
    blocks = []
    cin = 16
    for stage, cout in enumerate((16, 32, 64)):
        for b in range(3):
            stride = 2 if (stage > 0 and b == 0) else 1
            n = "s%db%d" % (stage, b)
            convs.append((n + "c1", cin, cout, 3, stride))
            convs.append((n + "c2", cout, cout, 3, 1))
            proj = None
            if stride != 1 or cin != cout:
                proj = n + "sc"
                convs.append((proj, cin, cout, 1, stride))
            blocks.append((n, cin, cout, stride, proj))
            cin = cout
    return convs, blocks, num_classes


def init_weights(seed, dt):
    convs, blocks, ncls = resnet20_spec()
    w = {}
    for i, (n, ci, co, k, s) in enumerate(convs):
        lim = float(np.sqrt(6.0 / (ci * k * k)))
        w[n] = hp.uniform(seed + i, (co, ci, k, k), -lim, lim).astype(hp.np_dtype(dt))
    w["fc"] = hp.uniform(seed + 99, (ncls, 64), -0.3, 0.3).astype(hp.np_dtype(dt))
    return w


class ResNetStep:
    """Device buffers, argument structs and the call sequence of one training step on `ns` samples."""

    def __init__(self, pkg, lib, torch, dt, ns, weights, lr=0.01, norm=False, fused=False, stats=False, post=False, pre=False, head=False):
        """`fused` (with `norm`): ReLU, the residual sum and the sum of a tensor's two incoming gradients run inside
        the normalisation calls (ptl_batch_norm_fused_*) instead of as element-wise calls of their own and the backward
        calls defer the additions of their weight gradients to one flush; with `stats` the forward convolutions also
        leave the sums the normalisation behind them needs (ptl_conv2d_*_fw_batched_stats), which then runs one launch
        instead of two; with `post` (and `stats`) the backward calls of the convolutions also form the gradient the
        normalisation in front of them starts from, and its sums (ptl_conv2d_*_bw_batched_deferred_post,
        ptl_batch_norm_fused_*_bw_stats): that normalisation's backward pass is one launch as well; with `pre` (and `stats`) the
        forward call of a convolution also stands for the forward call of the normalisation in front of it
        (ptl_conv2d_*_fw_batched_normed); with `head` pooling, classifier and loss run forward and backward in one
        call (ptl_pool_linear_loss_*_batched), the classifier's weight gradient deferred like the convolutions'."""
        self.pkg, self.lib, self.dt, self.ns, self.lr = pkg, lib, dt, ns, lr
        if fused:
            assert norm and (stats or not (post or pre))
            self.use_stats, self.use_post, self.use_pre, self.use_head = stats, post, pre, head
            return self._build_fused(torch, weights)
        assert not stats
        tdt = torch.float16 if dt == "fp16" else torch.float32
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
        z = lambda *s: torch.zeros(*s, dtype=tdt, device="cuda")
        convs, blocks, ncls = resnet20_spec()
        self.W = {n: dev(v) for n, v in weights.items()}
        self.dW = {n: z(*v.shape) for n, v in weights.items()}
        self.keep = []
        self.G, self.dG, self.Bt, self.dBt = {}, {}, {}, {}  # scale / shift of the normalisation layers
        eps = torch.full((1,), 1e-5, dtype=tdt, device="cuda")
        self.fw, self.bw = [], []  # lists of (function name, struct, extra args)
        self.conv_layers, self.norm_layers = [], []  # the tensors each such layer reads and writes (for per-layer checks)
        spec = {n: (ci, co, k, s) for n, ci, co, k, s in convs}
        L = lambda name: name.replace("DT", dt)

        def conv(name, x, dx, H):
            ci, co, k, s = spec[name]
            Ho = (H + 2 * (k // 2) - k) // s + 1
            y, dy = z(ns, co, Ho, Ho), z(ns, co, Ho, Ho)
            p = k // 2
            # strided layers: 32 + 2 - 3 is odd, which the reference's im2col route rejects; its naive-kernel route
            # (USE_IM2COL = 0, lib/sources/pulp_conv_naive_fp32.c:520) takes any stride, and so does this library's
            a, kp = hp.conv2d_args(pkg, x, dx, self.W[name], self.dW[name], y, dy, ci, H, H, co, k, k, Ho, Ho,
                                   (p, p, p, p), (s, s), 0, 1 if s == 1 else 0)
            self.keep.append(kp)
            self.conv_layers.append(dict(name=name, x=x, dx=dx, w=self.W[name], dw=self.dW[name], y=y, dy=dy,
                                         stride=s, pad=p))
            fw = [(L("ptl_conv2d_DT_fw_batched"), a, (ns,))]
            bw = [(L("ptl_conv2d_DT_wg_batched"), a, (ns,))]
            if dx is not None:
                bw.append((L("ptl_conv2d_DT_ig_batched"), a, (ns,)))
            if norm:
                self.G[name], self.Bt[name] = torch.ones(co, dtype=tdt, device="cuda"), z(co)
                self.dG[name], self.dBt[name] = z(co), z(co)
                n_, dn_ = z(ns, co, Ho, Ho), z(ns, co, Ho, Ho)
                na, kp = hp.batch_norm_args(pkg, y, n_, self.G[name], self.Bt[name], eps, ns, co, Ho, Ho, dy, dn_,
                                            self.dG[name], self.dBt[name])
                self.keep.append(kp)
                self.norm_layers.append(dict(name=name, x=y, dx=dy, y=n_, dy=dn_, g=self.G[name], b=self.Bt[name],
                                             dg=self.dG[name], db=self.dBt[name]))
                fw.append((L("ptl_batch_norm_DT_fw"), na, ()))
                bw.insert(0, (L("ptl_batch_norm_DT_bw"), na, ()))
                y, dy = n_, dn_
            return fw, bw, y, dy, Ho

        def relu(x, dx):
            y, dy = z(*x.shape), z(*x.shape)
            a, kp = hp.act_args(pkg, x, dx, y, dy, int(np.prod(x.shape[1:])))
            self.keep.append(kp)
            return a, y, dy

        self.x, self.dx0 = z(ns, 3, 32, 32), None
        f, first_bw, t, dt_, H = conv("stem", self.x, None, 32)  # the stem needs no input gradient
        self.fw += f
        ra, t, dt_ = relu(t, dt_)
        self.fw.append((L("ptl_relu_DT_batched"), ra, (ns, 0)))
        first_bw.insert(0, (L("ptl_relu_DT_batched"), ra, (ns, 1)))
        bw_blocks = []
        for (n, ci, co, stride, proj) in blocks:
            xin, dxin, Hin = t, dt_, H
            f1, b1, y1, dy1, H = conv(n + "c1", xin, dxin, Hin)
            r1, a1, da1 = relu(y1, dy1)
            f2, b2, y2, dy2, H = conv(n + "c2", a1, da1, H)
            seq = f1 + [(L("ptl_relu_DT_batched"), r1, (ns, 0))] + f2
            if proj:
                # the projection's input gradient must be ADDED to the main branch's: it gets its own buffer
                dproj = z(*xin.shape)
                fs, bs, ys, dys, _ = conv(proj, xin, dproj, Hin)
                seq += fs
                skip, dskip = ys, dys
            else:
                skip, dskip = xin, dxin
            s_, ds_ = z(*y2.shape), z(*y2.shape)
            sk, kp = hp.skip_args(pkg, skip, dskip, y2, dy2, s_, ds_, int(np.prod(y2.shape[1:])))
            self.keep.append(kp)
            r2, t, dt_ = relu(s_, ds_)
            seq += [(L("ptl_residual_DT_batched"), sk, (ns, 0)), (L("ptl_relu_DT_batched"), r2, (ns, 0))]
            self.fw += seq
            b = [(L("ptl_relu_DT_batched"), r2, (ns, 1)),            # ds = relu'(s) * dt
                 (L("ptl_residual_DT_batched"), sk, (ns, 2))]         # dy2 = ds
            b += b2 + [(L("ptl_relu_DT_batched"), r1, (ns, 1))] + b1  # ... dxin = main branch
            if proj:
                add, kp = hp.skip_args(pkg, dxin, dxin, dproj, dproj, dproj, dproj, int(np.prod(xin.shape[1:])))
                self.keep.append(kp)
                # dys = ds (copy through a residual-backward call on a view of the projection output)
                cp, kp2 = hp.skip_args(pkg, ys, dys, ys, dys, s_, ds_, int(np.prod(y2.shape[1:])))
                self.keep.append(kp2)
                b += [(L("ptl_residual_DT_batched"), cp, (ns, 2))] + bs + [self._vect_sum(dxin, dproj)]  # dxin += dproj
            else:
                b.append((L("ptl_residual_DT_batched"), sk, (ns, 1)))  # dxin += ds (identity shortcut)
            # what the shortcut adds to the buffer the first convolution's input gradient was written to
            next(l for l in self.conv_layers if l["name"] == n + "c1")["dx_extra"] = dproj if proj else ds_
            bw_blocks.append(b)
        pooled, dpooled = z(ns, 64), z(ns, 64)
        pa, kp = hp.pool_args(pkg, t, dt_, pooled, dpooled, 64, H, H, 1, 1, H, H, H, H)
        self.keep.append(kp)
        self.logits, dlogits = z(ns, ncls), z(ns, ncls)
        self.pooled, self.dpooled, self.dlogits = pooled, dpooled, dlogits
        la, kp = hp.linear_args(pkg, pooled, dpooled, self.W["fc"], self.dW["fc"], self.logits, dlogits, 64, ncls)
        self.keep.append(kp)
        self.target, self.loss = z(ns, ncls), z(ns)
        ca, kp = hp.loss_args(pkg, self.logits, dlogits, self.target, self.loss, ncls)
        self.keep.append(kp)
        self.fw += [(L("ptl_avgpool_DT_batched"), pa, (ns, 0)), (L("ptl_linear_DT_fw_batched"), la, (ns,)),
                    (L("ptl_cross_entropy_DT_batched"), ca, (ns, 0))]
        self.bw = [(L("ptl_cross_entropy_DT_batched"), ca, (ns, 1)), (L("ptl_linear_DT_bw_batched"), la, (ns,)),
                   (L("ptl_avgpool_DT_batched"), pa, (ns, 1))]
        for b in reversed(bw_blocks):
            self.bw += b
        self.bw += first_bw
        # one update call for all parameter tensors (the per-tensor call of the reference, once per struct)
        opts = []
        for n in self.W:
            o, kp = hp.optim_args(pkg, dt, self.W[n], self.dW[n], None, None, lr, 0.0)
            self.keep.append(kp)
            opts.append(o)
        for n in self.G:  # scale and shift of a normalisation layer share a struct
            o, kp = hp.optim_args(pkg, dt, self.G[n], self.dG[n], self.Bt[n], self.dBt[n], lr, 0.0)
            self.keep.append(kp)
            opts.append(o)
        table = (type(opts[0]) * len(opts))(*opts)
        self.opt = [(L("ptl_gradient_descent_DT_multi"), table, (len(opts),))]

    def _build_fused(self, torch, weights):
        pkg, dt, ns = self.pkg, self.dt, self.ns
        tdt = torch.float16 if dt == "fp16" else torch.float32
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
        z = lambda *s: torch.zeros(*s, dtype=tdt, device="cuda")
        convs, blocks, ncls = resnet20_spec()
        self.W = {n: dev(v) for n, v in weights.items()}
        self.dW = {n: z(*v.shape) for n, v in weights.items()}
        self.keep, self.G, self.dG, self.Bt, self.dBt = [], {}, {}, {}, {}
        self.conv_layers, self.norm_layers = [], []
        eps = torch.full((1,), 1e-5, dtype=tdt, device="cuda")
        spec = {n: (ci, co, k, s) for n, ci, co, k, s in convs}
        L = lambda name: name.replace("DT", dt)

        self.stats = {}  # per convolution: the struct its forward call fills and its normalisation reads
        self.grad_stats = {}  # per normalisation: the struct the backward call of the convolution behind it fills
        self.wg_buf = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
        self.wg_batch = pkg.WgBatch()
        self.wg_batch.buf, self.wg_batch.bytes = self.wg_buf.data_ptr(), self.wg_buf.numel()

        def conv(name, x, dx, H, post=None, pre=None):
            """The convolution alone: (forward call, backward calls, output, its gradient, output size).  `post`:
            (ptl_grad_post, ptl_norm_stats) of the normalisation in front of it; `pre`: that normalisation's forward
            call, which this layer's forward call then includes."""
            ci, co, k, s = spec[name]
            p = k // 2
            Ho = (H + 2 * p - k) // s + 1
            y, dy = z(ns, co, Ho, Ho), z(ns, co, Ho, Ho)
            a, kp = hp.conv2d_args(pkg, x, dx, self.W[name], self.dW[name], y, dy, ci, H, H, co, k, k, Ho, Ho,
                                   (p, p, p, p), (s, s), 0, 1 if s == 1 else 0)
            self.keep.append(kp)
            # weight and input gradient in one call (the stem needs no input gradient); the additions that complete
            # the weight gradients of the small layers wait for one flush behind the backward pass
            # (no input gradient: the backward call with skip_in_grad set is the weight-gradient step alone)
            a.skip_in_grad = 0 if dx is not None else 1
            bw = [(L("ptl_conv2d_DT_bw_batched_deferred"), a, (ns, self.wg_batch))]
            if post is not None:
                bw = [(L("ptl_conv2d_DT_bw_batched_deferred_post"), a, (ns, self.wg_batch, post[0], post[1]))]
            if not self.use_stats:
                return (L("ptl_conv2d_DT_fw_batched"), a, (ns,)), bw, y, dy, Ho
            # the forward call leaves the sums of its output for the normalisation behind it
            st = pkg.NormStats()
            part = torch.zeros(1 << 16, dtype=torch.float32, device="cuda")
            st.part, st.bytes = part.data_ptr(), part.numel() * 4
            self.stats[name] = st
            self.keep.append(part)
            if pre is not None:
                return (L("ptl_conv2d_DT_fw_batched_normed"), a, (ns, st, pre[1], pre[2][0], pre[2][1])), bw, y, dy, Ho
            return (L("ptl_conv2d_DT_fw_batched_stats"), a, (ns, st)), bw, y, dy, Ho

        def norm(name, y, dy, Ho, relu, skip=None, out_diff=None, out=None):
            """out = [relu](bn(y) [+ skip]); returns the calls, out, its gradient buffer and the fusion struct (whose
            skip_diff / diff2 the caller fills in once the tensors exist) - with `post` a triple of that struct, the
            ptl_grad_post and the ptl_norm_stats for the backward call of the convolution that reads `out`."""
            co = spec[name][1]
            self.G[name], self.Bt[name] = torch.ones(co, dtype=tdt, device="cuda"), z(co)
            self.dG[name], self.dBt[name] = z(co), z(co)
            out = out if out is not None else z(ns, co, Ho, Ho)
            dout = out_diff if out_diff is not None else z(ns, co, Ho, Ho)
            na, kp = hp.batch_norm_args(pkg, y, out, self.G[name], self.Bt[name], eps, ns, co, Ho, Ho, dy, dout,
                                        self.dG[name], self.dBt[name])
            f = pkg.NormFusion()
            f.relu = relu
            f.skip = pkg.addr(skip)
            self.keep += [kp, f, skip]
            fw = (L("ptl_batch_norm_fused_DT_fw_stats"), na, (f, self.stats[name])) if self.use_stats else (L("ptl_batch_norm_fused_DT_fw"), na, (f,))
            if self.use_post and out_diff is None:
                # the gradient of the sum is formed in place, by the convolution behind or (where that one leaves it
                # to this call) here
                f.skip_diff = pkg.addr(dout)
                po, gs = pkg.GradPost(), pkg.NormStats()
                po.mask, po.x = (pkg.addr(out) if relu else None), pkg.addr(y)
                part = torch.zeros(1 << 16, dtype=torch.float32, device="cuda")
                gs.part, gs.bytes = part.data_ptr(), part.numel() * 4
                self.keep += [po, gs, part]
                self.grad_stats[name] = gs
                return fw, (L("ptl_batch_norm_fused_DT_bw_stats"), na, (f, self.stats[name], gs)), out, dout, (f, po, gs)
            return fw, (L("ptl_batch_norm_fused_DT_bw"), na, (f,)), out, dout, f

        self.x = z(ns, 3, 32, 32)
        cf, cb, y, dy, H = conv("stem", self.x, None, 32)
        nf, nb, t, dt_, fus = norm("stem", y, dy, H, 1)
        post, pre = self.use_post, self.use_pre
        # (pending: the forward call of a normalisation that the next convolution's call will stand for)
        self.fw, pending = ([cf], nf) if pre else ([cf, nf], None)
        first_bw = [nb] + cb
        bw_blocks = []
        for (n, ci, co, stride, proj) in blocks:
            xin, dxin, Hin, fus_in = t, dt_, H, fus
            c1f, c1b, y1, dy1, H = conv(n + "c1", xin, dxin, Hin, fus_in[1:] if post else None, pending)
            n1f, n1b, a1, da1, fus1 = norm(n + "c1", y1, dy1, H, 1)
            c2f, c2b, y2, dy2, H = conv(n + "c2", a1, da1, H, fus1[1:] if post else None, n1f if pre else None)
            seq = [c1f, c2f] if pre else [c1f, n1f, c2f]
            # gradient of the sum = gradient of the shortcut branch (in place in the gradient of the block's output
            # when the convolution behind the block forms it)
            ds_ = None if post else z(*y2.shape)
            if proj:
                dproj = z(*xin.shape)
                csf, csb, ysr, dysr, _ = conv(proj, xin, dproj, Hin)
                # the projection's normalisation (no ReLU, nothing added) reads the gradient of the sum as the
                # gradient of its output
                nsf, nsb, ys = None, None, z(*y2.shape)
                skip = ys
            else:
                skip = xin
            n2f, n2b, t, dt_, fus = norm(n + "c2", y2, dy2, H, 1, skip=skip)
            if post:
                ds_ = dt_
            else:
                fus.skip_diff = pkg.addr(ds_)
            self.keep.append(ds_)
            if proj:
                nsf, nsb, _, _, _ = norm(proj, ysr, dysr, H, 0, out_diff=ds_, out=ys)
                seq += [csf, nsf]
            if pre:
                pending = n2f
            else:
                seq.append(n2f)
            self.fw += seq
            add = dproj if proj else ds_  # the block's input gets its gradient from c1 and from the shortcut
            if post:
                # (the projection's backward pass first: c1's call adds its input gradient)
                b = [n2b] + c2b + [n1b] + ([nsb] + csb if proj else []) + c1b
                fus_in[0].diff2 = fus_in[1].add = pkg.addr(add)
            else:
                b = [n2b] + c2b + [n1b] + c1b + ([nsb] + csb if proj else [])
                fus_in.diff2 = pkg.addr(add)
            self.keep.append(add)
            bw_blocks.append(b)
        if pending is not None:
            self.fw.append(pending)
        self._tail(torch, t, dt_, H, bw_blocks, first_bw, ncls)

    def _tail(self, torch, t, dt_, H, bw_blocks, first_bw, ncls):
        """Global average pooling, classifier, loss, the backward order and the update call."""
        pkg, dt, ns = self.pkg, self.dt, self.ns
        tdt = torch.float16 if dt == "fp16" else torch.float32
        z = lambda *s: torch.zeros(*s, dtype=tdt, device="cuda")
        L = lambda name: name.replace("DT", dt)
        pooled, dpooled = z(ns, 64), z(ns, 64)
        pa, kp = hp.pool_args(pkg, t, dt_, pooled, dpooled, 64, H, H, 1, 1, H, H, H, H)
        self.keep.append(kp)
        self.logits, dlogits = z(ns, ncls), z(ns, ncls)
        self.pooled, self.dpooled, self.dlogits = pooled, dpooled, dlogits
        la, kp = hp.linear_args(pkg, pooled, dpooled, self.W["fc"], self.dW["fc"], self.logits, dlogits, 64, ncls)
        self.keep.append(kp)
        self.target, self.loss = z(ns, ncls), z(ns)
        ca, kp = hp.loss_args(pkg, self.logits, dlogits, self.target, self.loss, ncls)
        self.keep.append(kp)
        if getattr(self, "use_head", False):
            self.fw += [(L("ptl_pool_linear_loss_DT_batched"), pa, (la, ca, ns, self.wg_batch))]
            self.bw = []
        else:
            self.fw += [(L("ptl_avgpool_DT_batched"), pa, (ns, 0)), (L("ptl_linear_DT_fw_batched"), la, (ns,)),
                        (L("ptl_cross_entropy_DT_batched"), ca, (ns, 0))]
            self.bw = [(L("ptl_cross_entropy_DT_batched"), ca, (ns, 1)), (L("ptl_linear_DT_bw_batched"), la, (ns,)),
                       (L("ptl_avgpool_DT_batched"), pa, (ns, 1))]
        for b in reversed(bw_blocks):
            self.bw += b
        self.bw += first_bw
        if hasattr(self, "wg_batch"):
            self.bw.append((L("ptl_conv2d_DT_wg_flush"), self.wg_batch, ()))
        opts = []
        for n in self.W:
            o, kp = hp.optim_args(pkg, dt, self.W[n], self.dW[n], None, None, self.lr, 0.0)
            self.keep.append(kp)
            opts.append(o)
        for n in self.G:
            o, kp = hp.optim_args(pkg, dt, self.G[n], self.dG[n], self.Bt[n], self.dBt[n], self.lr, 0.0)
            self.keep.append(kp)
            opts.append(o)
        table = (type(opts[0]) * len(opts))(*opts)
        self.opt = [(L("ptl_gradient_descent_DT_multi"), table, (len(opts),))]

    def _vect_sum(self, acc, term):
        """acc += term through the reference-named vect_sum entry point (lib/sources/pulp_train_utils_fp32.c:208)."""
        a = self.pkg.VectSumArgs()
        a.op_1, a.op_2, a.dest, a.size = self.pkg.addr(acc), self.pkg.addr(term), self.pkg.addr(acc), acc.numel()
        self.keep.append((acc, term))
        return ("vect_sum" if self.dt == "fp32" else "vect_sum_fp16", a, None)

    def _run(self, seq):
        for name, a, extra in seq:
            if extra is None:  # reference-named void entry point
                getattr(self.lib, name)(ctypes.byref(a))
                rc = self.lib.ptl_last_status()
            else:
                rc = getattr(self.lib, name)(ctypes.byref(a), *[ctypes.byref(e) if isinstance(e, ctypes.Structure) else e
                                                                 for e in extra])
            if rc != 0:
                raise RuntimeError("%s failed: %s" % (name, self.lib.ptl_last_error().decode()))

    def step(self, update=True):
        self._run(self.fw)
        self._run(self.bw)
        if update:
            self._run(self.opt)

    def launches(self):
        return len(self.fw) + len(self.bw) + len(self.opt)
