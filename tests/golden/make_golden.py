"""Writes the golden fixtures of tests/golden/*.npz.

The reference commits no golden numbers: each of its tests generates them at build time by running a torch
module on closed-form inputs (tests/test_conv2d_fp32/utils/GM.py:250-263,306-365,
tests/test_conv_pw_dw_fp32/utils/GM.py:45-56,97-102, tests/test_linear_fp32/utils/GM.py:78-99,
tests/test_matmul/utils/GM.py:81-99).  This script restates those closed-form inputs and evaluates the same
library routines (torch conv2d / linear / mm with autograd and an MSE loss) in float64; nothing from the
reference is imported or executed.  Outputs are stored as float64 so that both the fp32 and the fp16 paths can
be compared with them.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
F64 = torch.float64


def conv2d_case(Ci=8, Co=8, H=8, W=8, K=3, pad=0, stride=1):
    c, h, w = np.meshgrid(np.arange(Ci), np.arange(H), np.arange(W), indexing="ij")
    x = 1e-3 + (c + h - w) * (c + h + w) * 1e-5
    o, i, hk, wk = np.meshgrid(np.arange(Co), np.arange(Ci), np.arange(K), np.arange(K), indexing="ij")
    wt = (o + i + hk + wk) * 0.01
    Ho = (H - K + 2 * pad) // stride + 1
    Wo = (W - K + 2 * pad) // stride + 1
    label = np.broadcast_to(1.0 + np.arange(Wo) * 1e-3, (Co, Ho, Wo)).copy()
    tx = torch.tensor(x, dtype=F64)[None].requires_grad_()
    tw = torch.tensor(wt, dtype=F64).requires_grad_()
    ty = F.conv2d(tx, tw, padding=pad, stride=stride)
    ty.retain_grad()
    loss = F.mse_loss(ty, torch.tensor(label, dtype=F64)[None])
    loss.backward()
    return dict(x=x, w=wt, label=label, y=ty.detach()[0].numpy(), dy=ty.grad[0].numpy(), dw=tw.grad.numpy(),
                dx=tx.grad[0].numpy(), geom=np.array([Ci, Co, H, W, K, pad, stride]))


def pw_dw_case(C=8, Co=8, H=8, W=8, K=3):
    """Depthwise KxK (no padding) followed by pointwise C -> Co, label 1, MSE loss through both."""
    c, h, w = np.meshgrid(np.arange(C), np.arange(H), np.arange(W), indexing="ij")
    x = 1e-3 + (c + h - w) * (c + h + w) * 1e-5
    ch, hk, wk = np.meshgrid(np.arange(C), np.arange(K), np.arange(K), indexing="ij")
    wdw = (ch + hk + wk) * 0.01
    co, ci = np.meshgrid(np.arange(Co), np.arange(C), indexing="ij")
    wpw = (co * ci + 1) * 0.01
    tx = torch.tensor(x, dtype=F64)[None].requires_grad_()
    tdw = torch.tensor(wdw, dtype=F64)[:, None].requires_grad_()
    tpw = torch.tensor(wpw, dtype=F64)[:, :, None, None].requires_grad_()
    mid = F.conv2d(tx, tdw, groups=C)
    mid.retain_grad()
    out = F.conv2d(mid, tpw)
    out.retain_grad()
    loss = F.mse_loss(out, torch.ones_like(out))
    loss.backward()
    return dict(x=x, wdw=wdw, wpw=wpw, mid=mid.detach()[0].numpy(), out=out.detach()[0].numpy(),
                dout=out.grad[0].numpy(), dmid=mid.grad[0].numpy(), dwpw=tpw.grad[:, :, 0, 0].numpy(),
                dwdw=tdw.grad[:, 0].numpy(), dx=tx.grad[0].numpy(), geom=np.array([C, Co, H, W, K]))


def linear_case(n_in=1024, n_out=8):
    x = np.full(n_in, 1e-5)
    w = 0.01 * (np.arange(n_in * n_out) + 1).reshape(n_out, n_in)
    tx = torch.tensor(x, dtype=F64).requires_grad_()
    tw = torch.tensor(w, dtype=F64).requires_grad_()
    ty = F.linear(tx, tw)
    ty.retain_grad()
    loss = F.mse_loss(ty, torch.ones_like(ty))
    loss.backward()
    return dict(x=x, w=w, y=ty.detach().numpy(), dy=ty.grad.numpy(), dw=tw.grad.numpy(), dx=tx.grad.numpy())


def matmul_case(N=32, K=32, M=32, div=1e8):
    i, j = np.meshgrid(np.arange(N), np.arange(K), indexing="ij")
    A = (1.0 + (i + j + 0.1)) / div
    i, j = np.meshgrid(np.arange(K), np.arange(M), indexing="ij")
    B = i * j + 0.1
    return dict(A=A, B=B, C=torch.mm(torch.tensor(A, dtype=F64), torch.tensor(B, dtype=F64)).numpy(),
                Ct=torch.mm(torch.tensor(A, dtype=F64), torch.tensor(B.T.copy(), dtype=F64).t()).numpy())


def main():
    np.savez_compressed(os.path.join(HERE, "conv2d_ref_default.npz"), **conv2d_case())
    np.savez_compressed(os.path.join(HERE, "conv2d_ref_pad1_stride2.npz"), **conv2d_case(H=9, W=9, pad=1, stride=2))
    np.savez_compressed(os.path.join(HERE, "pw_dw_ref_default.npz"), **pw_dw_case())
    np.savez_compressed(os.path.join(HERE, "linear_ref_default.npz"), **linear_case())
    np.savez_compressed(os.path.join(HERE, "matmul_ref_default.npz"), **matmul_case())


if __name__ == "__main__":
    main()
