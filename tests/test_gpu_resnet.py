"""A ResNet-20-shaped training step (19 3x3 convolutions, two strided 1x1 projections, ReLU, residual sums,
global average pooling, linear classifier, cross-entropy, gradient descent) assembled from the library's entry
points, against torch autograd in float64 on the same inputs."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import helpers as hp
import resnet_step as rs

pytestmark = pytest.mark.gpu


def torch_step(weights, x, target, lr, norm=False, stored=None, device="cpu"):
    """`stored`: the type every tensor that the library materialises is rounded to on the way forward (the
    rounding passes gradients through unchanged), so that a float64 reference sees the activations - and with
    them the ReLU masks - that an fp16 run sees."""
    q = (lambda t: t.to(stored).to(torch.float64)) if stored is not None else (lambda t: t)
    convs, blocks, ncls = rs.resnet20_spec()
    p = {n: torch.tensor(v.astype(np.float64), requires_grad=True, device=device) for n, v in weights.items()}
    if norm:
        for n, ci, co, k, s in convs:
            p["g:" + n] = torch.ones(co, dtype=torch.float64, requires_grad=True, device=device)
            p["b:" + n] = torch.zeros(co, dtype=torch.float64, requires_grad=True, device=device)

    def conv(t, n, **kw):
        y = q(F.conv2d(t, p[n], **kw))
        return q(F.batch_norm(y, None, None, p["g:" + n], p["b:" + n], training=True, eps=1e-5)) if norm else y

    t = F.relu(conv(torch.tensor(x.astype(np.float64), device=device), "stem", padding=1))
    for (n, ci, co, stride, proj) in blocks:
        y = conv(F.relu(conv(t, n + "c1", stride=stride, padding=1)), n + "c2", padding=1)
        sc = conv(t, proj, stride=stride) if proj else t
        t = F.relu(q(y + sc))
    logits = t.mean((2, 3)) @ p["fc"].t()
    loss = F.cross_entropy(logits, torch.tensor(target.astype(np.float64), device=device), reduction="none")
    loss.sum().backward()
    return logits.detach().cpu().numpy(), loss.detach().cpu().numpy(), {n: v.grad.cpu().numpy() for n, v in p.items()}, \
        {n: (v.detach() - lr * v.grad).cpu().numpy() for n, v in p.items()}


@pytest.mark.parametrize("dt,ns,tol", [("fp32", 3, 2e-4), ("fp16", 4, 8e-2)])
def test_resnet20_training_step(pkg, gpu, dt, ns, tol):
    lr = 0.01
    w = rs.init_weights(0x2E5E0, dt)
    x = hp.normal(0x2E5E1, (ns, 3, 32, 32)).astype(hp.np_dtype(dt))
    tgt = np.zeros((ns, 10), hp.np_dtype(dt))
    tgt[np.arange(ns), (3 * np.arange(ns)) % 10] = 1
    net = rs.ResNetStep(pkg, gpu, torch, dt, ns, w, lr)
    net.x.copy_(torch.from_numpy(x))
    net.target.copy_(torch.from_numpy(tgt))
    net.step(update=True)
    assert gpu.ptl_sync() == 0
    ref_logits, ref_loss, ref_grads, ref_new = torch_step(w, x, tgt, float(hp.np_dtype(dt)(lr)))
    assert hp.rel_l2(net.logits.cpu().numpy(), ref_logits) <= tol
    assert hp.rel_l2(net.loss.cpu().numpy(), ref_loss) <= tol
    # gradients: classifier, last and first stage, a projection, the stem (the deepest path)
    for n in ("fc", "s2b2c2", "s2b0sc", "s1b0c1", "s0b0c1", "stem"):
        assert hp.rel_l2(net.dW[n].cpu().numpy(), ref_grads[n]) <= tol, n
    for n in w:
        assert hp.rel_l2(net.W[n].cpu().numpy(), ref_new[n]) <= tol, n
    assert net.launches() > 130


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("dt,ns,tol", [("fp32", 6, 1e-3), ("fp16", 8, 1.5e-1)])
def test_resnet20_training_step_with_batch_norm(pkg, gpu, dt, ns, tol, fused):
    """The same step with batch normalisation after every convolution (BASELINE's ResNet-20 configuration).
    fp16: the reference sees fp16-rounded activations; what remains is the rounding of the stored gradients, which
    twenty normalised layers down are of the order of 1e-4 and keep few significant bits in fp16 (no loss scaling,
    as in the reference) - 7 to 10 % on the deepest weight gradients, and around 15 % on the gain and shift gradients
    of the stem's normalisation, the deepest sums of such values (just under or just over 15 % depending on which of
    two equivalent orders the normalisation's forward arithmetic takes: they get 20 %)."""
    lr = 0.01
    w = rs.init_weights(0x2E5F0, dt)
    x = hp.normal(0x2E5F1, (ns, 3, 32, 32)).astype(hp.np_dtype(dt))
    tgt = np.zeros((ns, 10), hp.np_dtype(dt))
    tgt[np.arange(ns), (3 * np.arange(ns)) % 10] = 1
    net = rs.ResNetStep(pkg, gpu, torch, dt, ns, w, lr, norm=True, fused=fused)
    net.x.copy_(torch.from_numpy(x))
    net.target.copy_(torch.from_numpy(tgt))
    net.step(update=True)
    assert gpu.ptl_sync() == 0
    ref_logits, ref_loss, ref_grads, ref_new = torch_step(w, x, tgt, float(hp.np_dtype(dt)(lr)), norm=True,
                                                          stored=torch.float16 if dt == "fp16" else None)
    assert hp.rel_l2(net.logits.cpu().numpy(), ref_logits) <= tol
    assert hp.rel_l2(net.loss.cpu().numpy(), ref_loss) <= tol
    for n in ("fc", "s2b2c2", "s2b0sc", "s1b0c1", "stem"):
        assert hp.rel_l2(net.dW[n].cpu().numpy(), ref_grads[n]) <= tol, n
    for n in ("s2b2c2", "s0b0c1", "stem"):
        tol_n = 2e-1 if dt == "fp16" and n == "stem" else tol
        assert hp.rel_l2(net.dG[n].cpu().numpy(), ref_grads["g:" + n]) <= tol_n, n
        assert hp.rel_l2(net.dBt[n].cpu().numpy(), ref_grads["b:" + n]) <= tol_n, n
        assert hp.rel_l2(net.G[n].cpu().numpy(), ref_new["g:" + n]) <= tol, n
    for n in w:
        assert hp.rel_l2(net.W[n].cpu().numpy(), ref_new[n]) <= tol, n
    assert net.launches() > (80 if fused else 170)


@pytest.mark.parametrize("dt,ns,tol", [("fp32", 6, 1e-3), ("fp16", 16, 5e-3)])
def test_resnet20_step_with_sums_from_the_convolutions(pkg, gpu, dt, ns, tol):
    """The fused step whose forward convolutions leave the sums for the normalisation behind them
    (ptl_conv2d_*_fw_batched_stats / ptl_batch_norm_fused_*_fw_stats) against the fused step whose normalisation
    layers form their own: every convolution of the network leaves its sums, and the step comes out the same to the
    rounding of the statistics (fp32: everything the step writes; fp16, where one flipped rounding of an activation
    moves the deepest gradients by per cent: the forward results)."""
    w = rs.init_weights(0x2E610, dt)
    x = hp.normal(0x2E611, (ns, 3, 32, 32)).astype(hp.np_dtype(dt))
    nets = []
    for stats in (False, True):
        net = rs.ResNetStep(pkg, gpu, torch, dt, ns, w, 0.01, norm=True, fused=True, stats=stats)
        net.x.copy_(torch.from_numpy(x))
        net.target.zero_()
        net.target[torch.arange(ns), (3 * torch.arange(ns)) % 10] = 1
        net.step(update=True)
        assert gpu.ptl_sync() == 0
        nets.append(net)
    own, given = nets
    # (in fp32 the filters of a 64-channel layer are too large for the small-layer kernels: those layers leave no
    # sums and their normalisation forms its own)
    valid = sum(st.valid for st in given.stats.values())
    assert len(given.stats) == 21 and (valid == 21 if dt == "fp16" else 14 <= valid < 21), valid
    assert own.launches() == given.launches()
    rel = lambda a, b: hp.rel_l2(a.float().cpu().numpy(), b.float().cpu().numpy())
    assert rel(given.logits, own.logits) <= tol
    assert rel(given.loss, own.loss) <= tol
    if dt == "fp32":
        for n in own.dW:
            assert rel(given.dW[n], own.dW[n]) <= tol, n
            assert rel(given.W[n], own.W[n]) <= tol, n
        for n in own.dG:
            assert rel(given.dG[n], own.dG[n]) <= tol, n
            assert rel(given.dBt[n], own.dBt[n]) <= tol, n


@pytest.mark.parametrize("dt,ns,tol", [("fp32", 6, 1e-3), ("fp16", 16, 5e-3)])
def test_resnet20_step_with_gradient_sums_from_the_convolutions(pkg, gpu, dt, ns, tol):
    """The step whose backward convolutions also form the gradient of the normalisation in front of them and its sums
    (ptl_conv2d_*_bw_batched_deferred_post / ptl_batch_norm_fused_*_bw_stats) against the step whose normalisation
    layers do that themselves: the same forward pass bit for bit, the unit-stride 3x3 layers leave their sums (the
    normalisation behind a stride-2 layer, a projection's and the last one form their own), and the gradients come
    out the same to the rounding of the statistics (fp32: everything the step writes; fp16, where one flipped
    rounding moves the deepest gradients by per cent: the last stage's)."""
    w = rs.init_weights(0x2E620, dt)
    x = hp.normal(0x2E621, (ns, 3, 32, 32)).astype(hp.np_dtype(dt))
    nets = []
    for post in (False, True):
        net = rs.ResNetStep(pkg, gpu, torch, dt, ns, w, 0.01, norm=True, fused=True, stats=True, post=post)
        net.x.copy_(torch.from_numpy(x))
        net.target.zero_()
        net.target[torch.arange(ns), (3 * torch.arange(ns)) % 10] = 1
        net.step(update=True)
        assert gpu.ptl_sync() == 0
        nets.append(net)
    own, given = nets
    assert torch.equal(own.logits, given.logits) and torch.equal(own.loss, given.loss)
    # 19 normalisation layers have a convolution behind them; two of those convolutions have stride 2
    valid = sum(st.valid for st in given.grad_stats.values())
    assert len(given.grad_stats) == 19 and (valid >= 16 if dt == "fp16" else 10 <= valid <= 18), valid
    print("gradient sums left by", valid, "of 19")
    assert own.launches() == given.launches()
    rel = lambda a, b: hp.rel_l2(a.float().cpu().numpy(), b.float().cpu().numpy())
    names = list(own.dW) if dt == "fp32" else ["fc", "s2b2c2", "s2b2c1", "s2b1c2"]
    for n in names:
        assert rel(given.dW[n], own.dW[n]) <= tol, n
        assert rel(given.W[n], own.W[n]) <= tol, n
    for n in (own.dG if dt == "fp32" else ["s2b2c2", "s2b2c1", "s2b1c2"]):
        assert rel(given.dG[n], own.dG[n]) <= tol, n
        assert rel(given.dBt[n], own.dBt[n]) <= tol, n


@pytest.mark.parametrize("dt,ns", [("fp32", 6), ("fp16", 16)])
def test_resnet20_step_with_the_normalisation_inside_the_forward_convolutions(pkg, gpu, dt, ns):
    """The step whose forward convolution calls stand for the normalisation in front of them as well
    (ptl_conv2d_*_fw_batched_normed) against the step that calls the two one after the other: 18 calls fewer, and
    every tensor the step writes bit for bit the same."""
    w = rs.init_weights(0x2E630, dt)
    x = hp.normal(0x2E631, (ns, 3, 32, 32)).astype(hp.np_dtype(dt))
    nets = []
    for pre in (False, True):
        net = rs.ResNetStep(pkg, gpu, torch, dt, ns, w, 0.01, norm=True, fused=True, stats=True, post=True, pre=pre)
        net.x.copy_(torch.from_numpy(x))
        net.target.zero_()
        net.target[torch.arange(ns), (3 * torch.arange(ns)) % 10] = 1
        net.step(update=True)
        assert gpu.ptl_sync() == 0
        nets.append(net)
    two, one = nets
    assert two.launches() - one.launches() == 18
    assert torch.equal(two.logits, one.logits) and torch.equal(two.loss, one.loss)
    for n in two.dW:
        assert torch.equal(two.dW[n], one.dW[n]) and torch.equal(two.W[n], one.W[n]), n
    for n in two.dG:
        assert torch.equal(two.dG[n], one.dG[n]) and torch.equal(two.dBt[n], one.dBt[n]), n
        assert torch.equal(two.G[n], one.G[n]) and torch.equal(two.Bt[n], one.Bt[n]), n


@pytest.mark.parametrize("dt,ns,tol", [("fp32", 6, 1e-3), ("fp16", 16, 5e-3)])
def test_resnet20_step_with_pooling_classifier_and_loss_in_one_call(pkg, gpu, dt, ns, tol):
    """The step whose tail is one call (ptl_pool_linear_loss_*_batched) against the step with the six calls: five
    calls fewer, the same forward results up to the classifier's dot products, and gradients that agree to rounding
    (fp32: everything the step writes; fp16: the last stage's, as in the tests above)."""
    w = rs.init_weights(0x2E660, dt)
    x = hp.normal(0x2E661, (ns, 3, 32, 32)).astype(hp.np_dtype(dt))
    nets = []
    for head in (False, True):
        net = rs.ResNetStep(pkg, gpu, torch, dt, ns, w, 0.01, norm=True, fused=True, stats=True, post=True, pre=True, head=head)
        net.x.copy_(torch.from_numpy(x))
        net.target.zero_()
        net.target[torch.arange(ns), (3 * torch.arange(ns)) % 10] = 1
        net.step(update=True)
        assert gpu.ptl_sync() == 0
        nets.append(net)
    six, one = nets
    assert six.launches() - one.launches() == 5
    rel = lambda a, b: hp.rel_l2(a.float().cpu().numpy(), b.float().cpu().numpy())
    assert torch.equal(six.pooled, one.pooled)
    assert rel(one.logits, six.logits) <= tol and rel(one.loss, six.loss) <= tol
    names = list(six.dW) if dt == "fp32" else ["fc", "s2b2c2", "s2b2c1", "s2b1c2"]
    for n in names:
        assert rel(one.dW[n], six.dW[n]) <= tol, n
        assert rel(one.W[n], six.W[n]) <= tol, n
    for n in (six.dG if dt == "fp32" else ["s2b2c2", "s2b2c1", "s2b1c2"]):
        assert rel(one.dG[n], six.dG[n]) <= tol, n
        assert rel(one.dBt[n], six.dBt[n]) <= tol, n


@pytest.mark.parametrize("fused", [True, False, "stats", "post", "pre", "head"])
def test_training_step_replays_as_a_hip_graph(pkg, gpu, fused):
    """The whole step (92 or 178 library calls; "stats": the 92 with the sums of the convolutions' outputs formed by
    the convolutions) captured once into a HIP graph on a stream of the caller's and
    replayed: after the warm-up calls the library allocates nothing and records no memset node, so every replay -
    with eager library work and synchronisations between the replays - leaves bit for bit the parameters that the
    same steps leave when called one by one."""
    import ctypes
    ns, dt = 16, "fp16"
    side = torch.cuda.Stream()
    gpu.ptl_set_stream(ctypes.c_void_p(side.cuda_stream))
    try:
        with torch.cuda.stream(side):
            net = rs.ResNetStep(pkg, gpu, torch, dt, ns, rs.init_weights(0x2E600, dt), 0.01, norm=True, fused=bool(fused),
                                stats=fused in ("stats", "post", "pre", "head"), post=fused in ("post", "pre", "head"),
                                pre=fused in ("pre", "head"), head=fused == "head")
            net.x.copy_(torch.from_numpy(hp.normal(0x2E601, (ns, 3, 32, 32)).astype(np.float16)))
            net.target.zero_()
            net.target[torch.arange(ns), (3 * torch.arange(ns)) % 10] = 1
            for _ in range(2):  # (workspaces reach their size, kernel attributes are set)
                net.step()
            side.synchronize()
            params = dict(list(net.W.items()) + [("g:" + k, v) for k, v in net.G.items()] +
                          [("b:" + k, v) for k, v in net.Bt.items()])
            start = {n: v.clone() for n, v in params.items()}
            eager = []
            for _ in range(3):
                net.step()
                side.synchronize()
                eager.append({n: v.clone() for n, v in params.items()})
            for n in params:
                params[n].copy_(start[n])
            side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            net.step()
        other = torch.zeros(1 << 16, dtype=torch.float16, device="cuda")
        for k in range(3):
            graph.replay()
            torch.cuda.synchronize()
            for n in params:
                assert torch.equal(params[n], eager[k][n]), (k, n)
            with torch.cuda.stream(side):  # eager work of the library between the replays
                assert gpu.ptl_copy_bytes(ctypes.c_void_p(net.x.data_ptr()), ctypes.c_void_p(other.data_ptr()), 1 << 16) == 0
                side.synchronize()
    finally:
        gpu.ptl_set_stream(None)
        assert gpu.ptl_sync() == 0
