"""Elementwise (token-level) masks of the shapes users build (random, causal, sliding window, tile-constant with
stray tokens, many queries without keys, ragged documents with causal attention inside), forward and backward at
sequence lengths up to 4 200 (ragged or not), head dimensions 32 to 256, one mask for all heads or one per (batch, head).

The bar is the reference's own check, matmul + masked softmax (kernel-test.py:36-39), in fp32 on the GPU, and
torch.autograd through it for the gradients (the CPU oracle's backward is itself pinned against torch.autograd in
test_oracle_attention.py; at these sizes the oracle would take minutes per case).

Tolerances: rel-L2 1e-3 for O (3e-3 where O is typed bf16), LSE within 2e-3; gradients rel-L2 1e-3 (fp16), 3e-3 (bf16
inputs, fp32 results: O enters the backward rounded to bf16), 4e-3 (bf16-typed gradients)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

KINDS = ["rand", "causal", "window", "blocky", "rowsparse", "doc"]


def make_mask(rs, kind, Bm, Hm, N, keep, g, dev):
    i = torch.arange(N, device=dev)
    if kind == "rand":
        return torch.rand(Bm, Hm, N, N, generator=g, device=dev) < keep
    if kind == "causal":
        m = (i[:, None] >= i[None, :]).expand(Bm, Hm, N, N).clone()
        if rs.rand() < 0.5:
            m &= torch.rand(Bm, Hm, N, N, generator=g, device=dev) < max(keep, 0.3)
        return m
    if kind == "window":
        return ((i[:, None] - i[None, :]).abs() <= int(rs.randint(1, 700))).expand(Bm, Hm, N, N).clone()
    if kind == "blocky":        # tile-constant, given token by token, with stray tokens flipped
        nb = -(-N // 64)
        bm = torch.rand(Bm, Hm, nb, nb, generator=g, device=dev) < keep
        m = bm.repeat_interleave(64, 2).repeat_interleave(64, 3)[..., :N, :N].clone()
        m[..., ::7, ::5] ^= torch.rand(Bm, Hm, -(-N // 7), -(-N // 5), generator=g, device=dev) < 0.05
        return m
    if kind == "rowsparse":     # seven queries in ten attend to nothing
        rows = torch.rand(Bm, Hm, N, 1, generator=g, device=dev) < 0.3
        return (torch.rand(Bm, Hm, N, N, generator=g, device=dev) < keep) & rows
    cuts = np.sort(rs.choice(np.arange(1, N), size=min(N - 1, int(rs.randint(1, 12))), replace=False))
    doc = torch.from_numpy(np.searchsorted(cuts, np.arange(N), side="right")).to(dev)
    return ((doc[:, None] == doc[None, :]) & (i[:, None] >= i[None, :])).expand(Bm, Hm, N, N).clone()


def rel_l2(x, ref):
    x, ref = x.double(), ref.double()
    return float((x - ref).norm() / max(float(ref.norm()), 1e-30))


@pytest.mark.parametrize("seed", range(60))
def test_elementwise_structure(dev, seed):
    import fa2_custom_mask as fm
    rs = np.random.RandomState(seed)
    D = int(rs.choice([32, 64, 64, 128, 256]))
    dtype = torch.float16 if rs.rand() < 0.6 else torch.bfloat16
    B, H = int(rs.choice([1, 2])), int(rs.choice([1, 2, 3]))
    N = int(rs.randint(65, 4200))
    if rs.rand() < 0.4:
        N = (N // 64) * 64
    Bm, Hm = (B if rs.rand() < 0.4 else 1), (H if rs.rand() < 0.4 else 1)
    kind = KINDS[seed % len(KINDS)]
    keep = float(rs.choice([0.02, 0.1, 0.3, 0.6, 0.95]))
    out_fp32 = bool(rs.rand() < 0.5)
    print(dict(seed=seed, D=D, dtype=str(dtype), B=B, H=H, N=N, Bm=Bm, Hm=Hm, kind=kind, keep=keep, out_fp32=out_fp32),
          flush=True)
    m = make_mask(rs, kind, Bm, Hm, N, keep, torch.Generator(device=dev).manual_seed(seed), dev)
    gc = torch.Generator().manual_seed(seed)
    q, k, v, do = [torch.randn(B, H, N, D, generator=gc).to(dtype).to(dev) for _ in range(4)]
    sc = 1.0 / np.sqrt(D)
    o, lse, dq, dk, dv = fm.attention_forward_backward(q, k, v, m, sc, do, out_fp32=out_fp32)
    torch.cuda.synchronize()
    qf, kf, vf = [x.float().requires_grad_(True) for x in (q, k, v)]
    s = ((qf @ kf.transpose(-1, -2)) * sc).masked_fill(~m, float("-inf"))
    lse_ref = torch.logsumexp(s.detach(), dim=-1)
    p = torch.softmax(s, dim=-1)
    p = torch.where(torch.isnan(p), torch.zeros_like(p), p)      # queries without keys
    o_ref = p @ vf
    o_ref.backward(do.float())
    typed16 = not out_fp32
    o_bar = 3e-3 if (dtype == torch.bfloat16 and typed16) else 1e-3
    g_bar = 1e-3 if dtype == torch.float16 else (4e-3 if typed16 else 3e-3)
    none = torch.isinf(lse_ref)
    assert torch.equal(torch.isinf(lse), none)
    assert bool(torch.isfinite(o).all()) and bool((o[none] == 0).all())
    if (~none).any():
        assert float((lse[~none] - lse_ref[~none]).abs().max()) <= 2e-3
    assert rel_l2(o, o_ref.detach()) <= o_bar
    for name, got, ref in (("dq", dq, qf.grad), ("dk", dk, kf.grad), ("dv", dv, vf.grad)):
        assert bool(torch.isfinite(got).all()), name
        assert rel_l2(got, ref) <= g_bar or float(ref.abs().max()) < 1e-6, name
