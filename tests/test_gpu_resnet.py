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


def torch_step(weights, x, target, lr):
    convs, blocks, ncls = rs.resnet20_spec()
    p = {n: torch.tensor(v.astype(np.float64), requires_grad=True) for n, v in weights.items()}
    t = F.relu(F.conv2d(torch.tensor(x.astype(np.float64)), p["stem"], padding=1))
    for (n, ci, co, stride, proj) in blocks:
        y = F.conv2d(F.relu(F.conv2d(t, p[n + "c1"], stride=stride, padding=1)), p[n + "c2"], padding=1)
        sc = F.conv2d(t, p[proj], stride=stride) if proj else t
        t = F.relu(y + sc)
    logits = t.mean((2, 3)) @ p["fc"].t()
    loss = F.cross_entropy(logits, torch.tensor(target.astype(np.float64)), reduction="none")
    loss.sum().backward()
    return logits.detach().numpy(), loss.detach().numpy(), {n: v.grad.numpy() for n, v in p.items()}, \
        {n: (v.detach() - lr * v.grad).numpy() for n, v in p.items()}


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
    assert net.launches() > 150
