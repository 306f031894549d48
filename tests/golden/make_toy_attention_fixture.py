"""Writes tests/golden/toy_attention_fixture.npz: a seeded toy problem (B=1, H=2, N=128, D=64, fp16
inputs) with O, the natural-log LSE and dQ, dK, dV of the naive masked softmax attention
(kernel-test.py:37-40 of the reference: scores * sm_scale, masked_fill(-inf), softmax, @ v) computed in
float64 by torch on the CPU, gradients by torch.autograd.  Head 0 uses the block mask expanded as
kernel-test.py:18, head 1 an elementwise mask (token-level causal with a hole).  Independent of the
oracle and of the GPU path: both are checked against this file.

Run:  python tests/golden/make_toy_attention_fixture.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    g = torch.Generator().manual_seed(20240611)
    B, H, N, D = 1, 2, 128, 64
    q, k, v, do = [torch.randn(B, H, N, D, generator=g).to(torch.float16) for _ in range(4)]
    sm_scale = 0.125
    block = torch.tensor([[True, False], [True, True]])
    m0 = block.repeat_interleave(64, 0).repeat_interleave(64, 1)            # kernel-test.py:18
    m1 = torch.tril(torch.ones(N, N, dtype=torch.bool))
    m1[70:80, 10:40] = False
    m1[5, :] = False
    m1[5, 3] = True
    mask = torch.stack([m0, m1]).reshape(1, H, N, N)
    qd, kd, vd = [x.double().requires_grad_(True) for x in (q, k, v)]
    s = (qd @ kd.transpose(-1, -2)) * sm_scale                              # :37
    s = s.masked_fill(~mask, float("-inf"))                                 # :38
    p = torch.softmax(s, dim=-1)                                            # :39
    o = p @ vd                                                              # :40
    lse = torch.logsumexp(s, dim=-1)
    dq, dk, dv = torch.autograd.grad(o, (qd, kd, vd), do.double())
    np.savez_compressed(
        os.path.join(HERE, "toy_attention_fixture.npz"),
        q=q.numpy(), k=k.numpy(), v=v.numpy(), do=do.numpy(), sm_scale=np.float64(sm_scale),
        block_mask_head0=block.numpy(), mask=mask.numpy(),
        o=o.detach().float().numpy(), lse=lse.detach().float().numpy(),
        dq=dq.float().numpy(), dk=dk.float().numpy(), dv=dv.float().numpy())


if __name__ == "__main__":
    main()
