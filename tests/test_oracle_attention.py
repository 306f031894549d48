"""Pins the oracle's floating-point functions (CPU only) against library closed forms."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import bsattn_oracle as orc
from oracle import c_oracle


def rand_case(seed, B=1, H=2, nb=4, D=64, keep=0.5, dtype=np.float64):
    rng = np.random.default_rng(seed)
    N = nb * 64
    q, k, v = [rng.standard_normal((B, H, N, D)).astype(dtype) for _ in range(3)]
    mask = (rng.random((B, H, nb, nb)) < keep) | np.eye(nb, dtype=bool)
    return q, k, v, mask, 1.0 / np.sqrt(D)


def test_naive_dense_equals_sdpa():
    q, k, v, _, sc = rand_case(0)
    mask = np.ones((1, 2, 4, 4), dtype=bool)
    o = orc.naive_attention(q, k, v, mask, sc, dtype=np.float64)
    ref = F.scaled_dot_product_attention(torch.tensor(q), torch.tensor(k), torch.tensor(v), scale=sc)
    assert np.abs(o - ref.numpy()).max() < 1e-12


@pytest.mark.parametrize("seed", range(4))
def test_naive_masked_equals_sdpa_bool_mask(seed):
    q, k, v, mask, sc = rand_case(seed, H=3, nb=5)
    o, lse = orc.naive_attention(q, k, v, mask, sc, dtype=np.float64, return_lse=True, row_chunk=128)
    dense = torch.tensor(orc.expand_block_mask(mask))
    ref = F.scaled_dot_product_attention(torch.tensor(q), torch.tensor(k), torch.tensor(v),
                                         attn_mask=dense, scale=sc)
    assert np.abs(o - ref.numpy()).max() < 1e-12
    s = (torch.tensor(q) @ torch.tensor(k).transpose(-1, -2)) * sc           # kernel-test.py:37-38
    s = s.masked_fill(~dense, float("-inf"))
    assert np.abs(lse - torch.logsumexp(s, -1).numpy()).max() < 1e-12
    assert np.abs(orc.logsumexp(q, k, mask, sc, dtype=np.float64) - lse).max() == 0


def test_naive_closed_forms():
    q, k, v, mask, sc = rand_case(7, nb=6, keep=0.3)
    o = orc.naive_attention(q, k, np.full_like(v, 2.5), mask, sc, dtype=np.float64)
    assert np.abs(o - 2.5).max() < 1e-12                                     # rows of P sum to 1
    o = orc.naive_attention(q, np.zeros_like(k), v, mask, sc, dtype=np.float64)
    for h in range(2):
        for m in range(6):
            cols = np.nonzero(mask[0, h, m])[0]
            mean = np.concatenate([v[0, h, c * 64:(c + 1) * 64] for c in cols]).mean(0)
            assert np.abs(o[0, h, m * 64:(m + 1) * 64] - mean).max() < 1e-12
    eye = np.eye(6, dtype=bool)[None, None]                                  # block diagonal
    o = orc.naive_attention(q, k, v, eye, sc, dtype=np.float64)
    for m in range(6):
        sl = slice(m * 64, (m + 1) * 64)
        ref = F.scaled_dot_product_attention(torch.tensor(q[:, :, sl]), torch.tensor(k[:, :, sl]),
                                             torch.tensor(v[:, :, sl]), scale=sc).numpy()
        assert np.abs(o[:, :, sl] - ref).max() < 1e-12


def test_naive_empty_rows_defined():
    q, k, v, mask, sc = rand_case(2)
    mask[0, 1, 2, :] = False
    o, lse = orc.naive_attention(q, k, v, mask, sc, dtype=np.float64, return_lse=True)
    assert np.all(o[0, 1, 128:192] == 0) and np.all(np.isneginf(lse[0, 1, 128:192]))
    assert np.isfinite(o).all()


@pytest.mark.parametrize("seed", range(3))
def test_tiled_equals_naive(seed):
    """The online-softmax recurrence of fa2_fwd.py:146-196 reproduces the naive result."""
    q, k, v, mask, sc = rand_case(seed, B=2, nb=5, keep=0.4)
    groups, n_list = orc.build_groups_from_block_mask(mask)
    o, M, lse = orc.tiled_attention(q, k, v, groups, n_list, sc, dtype=np.float64)
    o_ref, lse_ref = orc.naive_attention(q, k, v, mask, sc, dtype=np.float64, return_lse=True)
    # the reference's log2(e) constant is truncated to 1.44269504 (fa2_fwd.py:150): ~6e-9 relative
    assert np.abs(o - o_ref).max() < 1e-8 and np.abs(lse - lse_ref).max() < 1e-7
    s = np.where(orc.expand_block_mask(mask), (q @ np.swapaxes(k, -1, -2)) * sc, -np.inf)
    assert np.abs(M - s.max(-1) * np.log2(np.e)).max() < 1e-6                # the reference's M: row max, base 2
    o32, _, _ = orc.tiled_attention(q, k, v, groups, n_list, sc, dtype=np.float32)
    assert np.abs(o32 - o_ref).max() < 1e-5


def test_tiled_order_invariance_and_p_rounding():
    q, k, v, mask, sc = rand_case(11, nb=6)
    groups, n_list = orc.build_groups_from_block_mask(mask)
    o1, _, _ = orc.tiled_attention(q, k, v, groups, n_list, sc, dtype=np.float64)
    rev = n_list.copy()
    for _, _, _, s, l in groups.tolist():
        rev[s:s + l] = n_list[s:s + l][::-1]
    o2, _, _ = orc.tiled_attention(q, k, v, groups, rev, sc, dtype=np.float64)
    assert np.abs(o1 - o2).max() < 1e-12
    o3, _, _ = orc.tiled_attention(q, k, v, groups, n_list, sc, dtype=np.float64, p_round=np.float16)
    assert 0 < np.abs(o1 - o3).max() < 2e-3                                  # fa2_fwd.py:189 costs ~1e-4


def test_c_naive_equals_numpy():
    q, k, v, mask, sc = rand_case(4, B=2, H=2, nb=4, dtype=np.float32)
    mask[1, 0, 1, :] = False
    o_ref, lse_ref = orc.naive_attention(q, k, v, mask, sc, dtype=np.float64, return_lse=True)
    o, lse = c_oracle.naive_fwd(q, k, v, mask, sc)
    assert np.abs(o - o_ref).max() < 2e-5
    fin = np.isfinite(lse_ref)
    assert np.array_equal(np.isfinite(lse), fin) and np.abs(lse[fin] - lse_ref[fin]).max() < 2e-5
    o2, _ = c_oracle.naive_fwd(q, k, v, mask[:1, :1], sc, row0=64, row1=128)  # shared mask, row sample
    ref2 = orc.naive_attention(q, k, v, mask[:1, :1], sc, dtype=np.float64)
    assert np.abs(o2[:, :, 64:128] - ref2[:, :, 64:128]).max() < 2e-5
    assert np.all(o2[:, :, :64] == 0)


def torch_grads(q, k, v, mask, sc, do):
    qt, kt, vt = [torch.tensor(x, requires_grad=True) for x in (q, k, v)]
    dense = torch.tensor(orc.expand_block_mask(mask))
    attn = (qt @ kt.transpose(-2, -1)) * sc                                   # kernel-test.py:37
    attn = attn.masked_fill(~dense, float("-inf"))                            # :38
    out = torch.softmax(attn, -1) @ vt                                        # :39-40
    return [g.numpy() for g in torch.autograd.grad(out, (qt, kt, vt), torch.tensor(do))], out.detach().numpy()


@pytest.mark.parametrize("seed", range(3))
def test_backward_equals_autograd(seed):
    q, k, v, mask, sc = rand_case(seed, B=1, H=2, nb=3, D=64)
    do = np.random.default_rng(seed + 100).standard_normal(q.shape)
    (dq_r, dk_r, dv_r), out = torch_grads(q, k, v, mask, sc, do)
    dq, dk, dv, delta = orc.attention_backward(q, k, v, mask, sc, do, dtype=np.float64)
    for a, b in ((dq, dq_r), (dk, dk_r), (dv, dv_r)):
        assert np.abs(a - b).max() < 1e-11
    assert np.abs(delta - (out * do).sum(-1)).max() < 1e-11                   # fa2_bwd.py:17


def test_backward_with_stored_output():
    """o_stored only replaces the O that delta is taken from.  Given the exact O the gradients are the autograd
    ones; given O + E the change is what the algebra fixes: delta' = delta + rowsum(E dO), dV unchanged,
    dQ' - dQ = -(P * rowsum(E dO)) K sm_scale and dK' - dK = -(P * rowsum(E dO))^T Q sm_scale, with P taken from
    torch's own softmax."""
    q, k, v, mask, sc = rand_case(5, B=1, H=2, nb=3, D=64)
    rng = np.random.default_rng(55)
    do = rng.standard_normal(q.shape)
    (dq_r, dk_r, dv_r), out = torch_grads(q, k, v, mask, sc, do)
    dq, dk, dv, delta = orc.attention_backward(q, k, v, mask, sc, do, dtype=np.float64, o_stored=out)
    for a, b in ((dq, dq_r), (dk, dk_r), (dv, dv_r)):
        assert np.abs(a - b).max() < 1e-11
    E = 0.01 * rng.standard_normal(q.shape)
    dq2, dk2, dv2, delta2 = orc.attention_backward(q, k, v, mask, sc, do, dtype=np.float64, o_stored=out + E)
    shift = (E * do).sum(-1)
    assert np.abs(delta2 - delta - shift).max() < 1e-11 and np.abs(dv2 - dv).max() == 0.0
    em = torch.tensor(mask).repeat_interleave(64, 2).repeat_interleave(64, 3)
    sm = torch.softmax((torch.tensor(q) @ torch.tensor(k).transpose(-1, -2) * sc).masked_fill(~em, float("-inf")), -1)
    corr = sm * torch.tensor(shift)[..., None]
    assert np.abs((dq2 - dq) + (corr @ torch.tensor(k)).numpy() * sc).max() < 1e-11
    assert np.abs((dk2 - dk) + (corr.transpose(-1, -2) @ torch.tensor(q)).numpy() * sc).max() < 1e-11


def test_backward_finite_differences():
    rng = np.random.default_rng(9)
    q, k, v, mask, sc = rand_case(9, B=1, H=1, nb=2, D=16)
    do = rng.standard_normal(q.shape)
    dq, dk, dv, _ = orc.attention_backward(q, k, v, mask, sc, do, dtype=np.float64)

    def loss(q_, k_, v_):
        return (orc.naive_attention(q_, k_, v_, mask, sc, dtype=np.float64) * do).sum()
    eps = 1e-6
    for arr, grad, which in ((q, dq, 0), (k, dk, 1), (v, dv, 2)):
        for _ in range(6):
            idx = tuple(rng.integers(0, s) for s in arr.shape)
            ap, am = arr.copy(), arr.copy()
            ap[idx] += eps; am[idx] -= eps
            args_p = [q, k, v]; args_m = [q, k, v]
            args_p[which] = ap; args_m[which] = am
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - grad[idx]) < 1e-6 * max(1.0, abs(fd))


def test_elementwise_mask_matches_sdpa_bool_mask():
    """An arbitrary elementwise mask (every row keeps at least one key) against torch's
    scaled_dot_product_attention with a boolean attn_mask, forward and gradients."""
    g = torch.Generator().manual_seed(5)
    B, H, N, D = 1, 2, 128, 16
    q, k, v, do = [torch.randn(B, H, N, D, generator=g, dtype=torch.float64) for _ in range(4)]
    m = torch.rand(1, H, N, N, generator=g) < 0.3
    m |= torch.eye(N, dtype=torch.bool)
    m[0, 0, 64:, :64] = False                     # an empty tile
    m[0, 1, :64, 64:] = True                      # a full tile
    qr, kr, vr = [x.clone().requires_grad_(True) for x in (q, k, v)]
    ref = torch.nn.functional.scaled_dot_product_attention(qr, kr, vr, attn_mask=m, scale=0.25)
    ref.backward(do)
    o, lse = orc.naive_attention(q.numpy(), k.numpy(), v.numpy(), m.numpy(), 0.25, dtype=np.float64, return_lse=True)
    assert np.abs(o - ref.detach().numpy()).max() < 1e-12
    s = (q @ k.transpose(-1, -2) * 0.25).masked_fill(~m, float("-inf"))
    assert np.abs(lse - torch.logsumexp(s, -1).numpy()).max() < 1e-12
    dq, dk, dv, _ = orc.attention_backward(q.numpy(), k.numpy(), v.numpy(), m.numpy(), 0.25, do.numpy(), dtype=np.float64)
    for got, want in ((dq, qr.grad), (dk, kr.grad), (dv, vr.grad)):
        assert np.abs(got - want.numpy()).max() < 1e-11


def test_elementwise_rows_without_keys_give_zero():
    g = torch.Generator().manual_seed(6)
    q, k, v = [torch.randn(1, 1, 64, 8, generator=g).numpy() for _ in range(3)]
    m = np.ones((1, 1, 64, 64), dtype=bool)
    m[0, 0, 5, :] = False
    o, lse = orc.naive_attention(q, k, v, m, 0.5, return_lse=True)
    assert np.all(o[0, 0, 5] == 0) and lse[0, 0, 5] == -np.inf and np.isfinite(lse[0, 0, 4])


def test_oracle_matches_committed_toy_fixture():
    """tests/golden/toy_attention_fixture.npz holds O, LSE and gradients of a seeded toy problem computed in
    float64 by torch (naive formula of kernel-test.py:37-40 + autograd), one head with a block mask and one
    with an elementwise mask."""
    import os
    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "toy_attention_fixture.npz"))
    q, k, v, do = [fx[n].astype(np.float32) for n in ("q", "k", "v", "do")]
    sc = float(fx["sm_scale"])
    o, lse = orc.naive_attention(q, k, v, fx["mask"], sc, return_lse=True)
    assert np.abs(o - fx["o"]).max() <= 2e-6 and np.abs(lse - fx["lse"]).max() <= 2e-6
    for got, name in zip(orc.attention_backward(q, k, v, fx["mask"], sc, do), ("dq", "dk", "dv")):
        assert np.abs(got - fx[name]).max() <= 2e-5, name
    # head 0 through the block form of its mask, numpy and C restatements
    bm = fx["block_mask_head0"].reshape(1, 1, 2, 2)
    o0 = orc.naive_attention(q[:, :1], k[:, :1], v[:, :1], bm, sc)
    assert np.abs(o0 - fx["o"][:, :1]).max() <= 2e-6
    oc, lc = c_oracle.naive_fwd(q[:, :1], k[:, :1], v[:, :1], bm, sc, 0, 128)
    assert np.abs(oc - fx["o"][:, :1]).max() <= 2e-6 and np.abs(lc - fx["lse"][:, :1]).max() <= 2e-6
    groups, n_list = orc.build_groups_from_block_mask(bm)
    ot = orc.tiled_attention(q[:, :1], k[:, :1], v[:, :1], groups, n_list, sc)
    ot = ot[0] if isinstance(ot, tuple) else ot
    assert np.abs(ot - fx["o"][:, :1]).max() <= 2e-6
