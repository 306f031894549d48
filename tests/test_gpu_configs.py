"""Parity at the full sizes of the benchmark configurations.  The oracle runs on sampled
row blocks (forward) or sampled heads (backward) so that the CPU side stays within seconds;
the rest of the output is covered by size-independent properties."""
import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from oracle import c_oracle
from helpers import make_qkv, uniform_block_mask, causal_block_mask, errors, f32, same_up_to_rounding

pytestmark = pytest.mark.gpu


def sampled_forward_check(dev, N, D, mask, seed, blocks):
    import fa2_custom_mask as fm
    q, k, v = make_qkv(1, 1, N, D, torch.float16, seed)
    sc = 1.0 / np.sqrt(D)
    o, lse = fm.flash_attention_custom_mask_lse(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), sc)
    o = o.float().cpu().numpy(); lse = lse.cpu().numpy()
    assert np.isfinite(o).all()
    qf, kf, vf = f32(q), f32(k), f32(v)
    for mb in blocks:
        r0, r1 = mb * 64, mb * 64 + 64
        o_ref, lse_ref = c_oracle.naive_fwd(qf, kf, vf, mask.numpy(), sc, r0, r1)
        d = o[0, 0, r0:r1] - o_ref[0, 0, r0:r1]
        ma = np.abs(d).max(); rl = np.linalg.norm(d) / np.linalg.norm(o_ref[0, 0, r0:r1])
        assert ma <= 2e-2 and rl <= 1e-3, (mb, ma, rl)
        assert np.abs(lse[0, 0, r0:r1] - lse_ref[0, 0, r0:r1]).max() <= 2e-3
    return q, k, v, o


@pytest.mark.parametrize("keep", [0.05, 0.1, 0.25, 0.5, 1.0])
def test_c3_n17536(dev, keep):
    nb = 274
    sampled_forward_check(dev, 17536, 64, uniform_block_mask(1, 1, nb, keep, 1236), 1236, [0, 1, 137, 272, 273])


@pytest.mark.parametrize("B,H,N,D", [(1, 2, 8192, 64), (2, 2, 8192, 64), (1, 4, 4096, 64), (1, 1, 8192, 128), (1, 2, 8192, 128)])
def test_dense_few_heads_ranges_dealt_by_phase(dev, B, H, N, D):
    """Dense masks with 2 or 4 heads in the launch: every head is cut into ranges that the workgroups take in the
    order of the launcher's range permutation (ranges of like phase on one XCD), as the single dense head of
    test_c3_n17536 is.  Sampled row blocks of every head against the oracle."""
    import fa2_custom_mask as fm
    nb = N // 64
    q, k, v = make_qkv(B, H, N, D, torch.float16, 1250 + B * H)
    mask = torch.ones(1, 1, nb, nb, dtype=torch.bool)
    sc = 1.0 / np.sqrt(D)
    o, lse = fm.flash_attention_custom_mask_lse(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), sc)
    o = o.float().cpu().numpy(); lse = lse.cpu().numpy()
    assert np.isfinite(o).all()
    for b in range(B):
        for h in range(H):
            qf, kf, vf = f32(q[b:b + 1, h:h + 1]), f32(k[b:b + 1, h:h + 1]), f32(v[b:b + 1, h:h + 1])
            for mb in (0, nb // 2, nb - 1):
                r0, r1 = mb * 64, mb * 64 + 64
                o_ref, lse_ref = c_oracle.naive_fwd(qf, kf, vf, mask.numpy(), sc, r0, r1)
                d = o[b, h, r0:r1] - o_ref[0, 0, r0:r1]
                assert np.abs(d).max() <= 2e-2 and np.linalg.norm(d) / np.linalg.norm(o_ref[0, 0, r0:r1]) <= 1e-3, (b, h, mb)
                assert np.abs(lse[b, h, r0:r1] - lse_ref[0, 0, r0:r1]).max() <= 2e-3


@pytest.mark.parametrize("keep", [0.1, 1.0])
def test_c4_n32000_block_causal(dev, keep):
    nb = 500
    mask = causal_block_mask(1, 1, nb, keep, 1237)
    q, k, v, o = sampled_forward_check(dev, 32000, 64, mask, 1237, [0, 1, 250, 499])
    # causality: changing the last key/value tile must leave every earlier row block unchanged
    import fa2_custom_mask as fm
    k2, v2 = k.clone(), v.clone()
    k2[0, 0, -64:] += 1.0; v2[0, 0, -64:] -= 1.0
    o2 = fm.flash_attention_custom_mask(q.to(dev), k2.to(dev), v2.to(dev), mask.to(dev), 0.125).float().cpu().numpy()
    assert same_up_to_rounding(o2[0, 0, :-64], o[0, 0, :-64])


def test_very_long_sequence_n262144(dev):
    """4096 row blocks: the row-pointer searches leave their one-load-per-lane form (binary search),
    and a range's column list no longer fits its LDS staging area.  Sparse mask (a band, a few random
    tiles and one long row block); forward on sampled row blocks, lists bit-exact."""
    import fa2_custom_mask as fm
    N, nb = 262144, 4096
    g = torch.Generator().manual_seed(1240)
    idx = torch.arange(nb)
    mask = ((idx[:, None] - idx[None, :]).abs() <= 2) | (torch.rand(nb, nb, generator=g) < 0.001)
    mask[2000, ::2] = True                       # 2048 + kept tiles in one row block
    mask[2001, :] = False                        # a row block without any
    mask = mask.reshape(1, 1, nb, nb)
    groups, n_list = fm.build_groups_from_block_mask(mask.to(dev))
    g_ref, n_ref = orc.build_groups_from_block_mask(mask.numpy())
    assert np.array_equal(groups.cpu().numpy(), g_ref) and np.array_equal(n_list.cpu().numpy(), n_ref)
    q, k, v, o = sampled_forward_check(dev, N, 64, mask, 1240, [0, 1, 1999, 2000, 2002, 4095])
    assert float(np.abs(o[0, 0, 2001 * 64:2002 * 64]).max()) == 0.0


def test_head_dim_256_row_lists_shared_by_workgroups(dev):
    """D = 256, one head, 128 row blocks: every row list is split over 8 workgroups whose fp32 parts a
    second kernel sums.  Rows with fewer tiles than parts (empty parts), a full row and an empty row."""
    nb = 128
    mask = uniform_block_mask(1, 1, nb, 0.04, 1241)
    mask[0, 0, 5, :] = True
    mask[0, 0, 6, :] = False
    mask[0, 0, 7, :] = False; mask[0, 0, 7, 100] = True
    q, k, v, o = sampled_forward_check(dev, nb * 64, 256, mask, 1241, [0, 5, 7, 64, 127])
    assert float(np.abs(o[0, 0, 6 * 64:7 * 64]).max()) == 0.0


@pytest.mark.parametrize("keep", [0.1, 1.0])
@pytest.mark.parametrize("route", ["elementwise", "reduced"])
def test_c2_dense_elementwise_mask_n6400(dev, keep, route):
    """C2: the mask arrives as a dense, tile-constant N x N bool tensor (kernel-test.py:18).  Both routes from it
    (taken as an elementwise mask; reduced to the block mask first) against the oracle on sampled row blocks,
    and the lists made from the reduced mask against the oracle's, bit for bit."""
    import fa2_custom_mask as fm
    N, nb = 6400, 100
    block = uniform_block_mask(1, 1, nb, keep, 1235)
    dense = block.to(dev).repeat_interleave(64, 2).repeat_interleave(64, 3)
    q, k, v = make_qkv(1, 1, N, 64, torch.float16, 1235)
    sc = 0.125
    m_in = dense if route == "elementwise" else fm.reduce_dense_mask(dense)
    if route == "reduced":
        groups, n_list = fm.build_groups_from_block_mask(m_in)
        g_ref, n_ref = orc.build_groups_from_block_mask(block.numpy())
        assert np.array_equal(groups.cpu().numpy(), g_ref) and np.array_equal(n_list.cpu().numpy(), n_ref)
    o, lse = fm.flash_attention_custom_mask_lse(q.to(dev), k.to(dev), v.to(dev), m_in, sc)
    o = o.float().cpu().numpy(); lse = lse.cpu().numpy()
    assert np.isfinite(o).all()
    qf, kf, vf = f32(q), f32(k), f32(v)
    for mb in (0, 1, 50, 98, 99):
        r0, r1 = mb * 64, mb * 64 + 64
        o_ref, lse_ref = c_oracle.naive_fwd(qf, kf, vf, block.numpy(), sc, r0, r1)
        d = o[0, 0, r0:r1] - o_ref[0, 0, r0:r1]
        assert np.abs(d).max() <= 2e-2 and np.linalg.norm(d) / np.linalg.norm(o_ref[0, 0, r0:r1]) <= 1e-3, mb
        assert np.abs(lse[0, 0, r0:r1] - lse_ref[0, 0, r0:r1]).max() <= 2e-3


def test_c5_fwd_bwd_bf16_d128(dev):
    """C5: B=2 H=16 N=8192 D=128 bf16, block-causal keep 0.25 shared across heads; O, LSE, dQ, dK,
    dV of two sampled heads against the oracle (fp32 outputs: the rel-L2 bar of 1e-3 is below
    what a bf16-typed result can meet), all heads against the bf16-typed run."""
    import fa2_custom_mask as fm
    B, H, N, D, nb = 2, 16, 8192, 128, 128
    q, k, v, do = make_qkv(B, H, N, D, torch.bfloat16, 1238, n=4)
    mask = causal_block_mask(1, 1, nb, 0.25, 1238)
    sc = 1.0 / np.sqrt(D)
    args = [x.to(dev) for x in (q, k, v)]
    o, lse, dq, dk, dv = fm.attention_forward_backward(*args, mask.to(dev), sc, do.to(dev), out_fp32=True)
    for (b, h) in ((0, 0), (1, 15)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        qh, kh, vh, doh = [f32(x[sl]) for x in (q, k, v, do)]
        o_r, lse_r = orc.naive_attention(qh, kh, vh, mask.numpy(), sc, return_lse=True)
        dq_r, dk_r, dv_r, _ = orc.attention_backward(qh, kh, vh, mask.numpy(), sc, doh)
        for name, got, ref in (("O", o, o_r), ("dQ", dq, dq_r), ("dK", dk, dk_r), ("dV", dv, dv_r)):
            ma, rl = errors(got[sl], ref)
            print("C5 head (%d,%d) %s: max-abs %.3e rel-L2 %.3e" % (b, h, name, ma, rl))
            assert ma <= 3e-2 and rl <= 1e-3
        assert np.abs(lse[sl].cpu().numpy() - lse_r).max() <= 2e-3
    o16, _, dq16, dk16, dv16 = fm.attention_forward_backward(*args, mask.to(dev), sc, do.to(dev), out_fp32=False)
    for a, b_ in ((o16, o), (dq16, dq), (dk16, dk), (dv16, dv)):
        assert a.dtype == torch.bfloat16
        assert errors(a, b_)[1] <= 3e-3                           # the same values up to bf16 rounding


def test_committed_toy_fixture(dev):
    """Forward, LSE and gradients against tests/golden/toy_attention_fixture.npz (float64 torch on the CPU):
    both heads through the elementwise mask, head 0 also through the block form of its mask."""
    import os
    import fa2_custom_mask as fm
    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "toy_attention_fixture.npz"))
    q, k, v, do = [torch.from_numpy(fx[n]).to(dev) for n in ("q", "k", "v", "do")]
    sc = float(fx["sm_scale"])
    mask = torch.from_numpy(fx["mask"]).to(dev)
    res = fm.attention_forward_backward(q, k, v, mask, sc, do, out_fp32=True)
    for got, name in zip(res, ("o", "lse", "dq", "dk", "dv")):
        ma, rl = errors(got, fx[name])
        print("%s max-abs %.3e rel-L2 %.3e" % (name, ma, rl))
        assert ma <= 2e-2 and rl <= 1e-3, name
    bm = torch.from_numpy(fx["block_mask_head0"]).reshape(1, 1, 2, 2).to(dev)
    res0 = fm.attention_forward_backward(q[:, :1], k[:, :1], v[:, :1], bm, sc, do[:, :1], out_fp32=True)
    for got, name in zip(res0, ("o", "lse", "dq", "dk", "dv")):
        ma, rl = errors(got, fx[name][:, :1])
        assert ma <= 2e-2 and rl <= 1e-3, name
