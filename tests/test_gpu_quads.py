"""GPU parity of the forward kernel that walks quads of row blocks (bsattn_quad_lists +
bsattn_fwd_quads, through the C ABI): the quad lists bit-exact against a numpy restatement (union of
the four rows' kept columns, ascending, with the membership bits), the attention against the CPU
oracle's naive fp32 masked softmax (kernel-test.py:37-40) to the tolerances of the forward tests:
max-abs 2e-2 / 3e-2, rel-L2 1e-3 (3e-3 for a bf16-typed output), LSE 2e-3 with the same -inf rows."""
import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from helpers import make_qkv, uniform_block_mask, causal_block_mask, errors, f32

pytestmark = pytest.mark.gpu


def quad_lists_restated(mask):
    Bm, Hm, nb, _ = mask.shape
    mm = mask.reshape(Bm * Hm, nb, nb)
    nq = (nb + 3) // 4
    ptr, entries = [0], []
    for mh in range(Bm * Hm):
        for qi in range(nq):
            rows = mm[mh, 4 * qi: 4 * qi + 4]
            cols = np.nonzero(rows.any(0))[0]
            entries.append([int(c) | (sum(int(rows[r, c]) << r for r in range(rows.shape[0])) << 16) for c in cols])
            ptr.append(ptr[-1] + len(cols))
    return ptr, entries


def run_case(dev, B, H, N, mask, dtype=torch.float16, seed=0, out_fp32=False):
    import fa2_custom_mask as fm
    q, k, v = make_qkv(B, H, N, 64, dtype, seed)
    sm_scale = 0.125
    lists = fm.block_mask_to_lists(mask.to(dev))
    qd = lists.quads()
    torch.cuda.synchronize()
    nb = N // 64
    ptr, entries = quad_lists_restated(mask.numpy())
    assert qd.quad_ptr.cpu().tolist() == ptr
    ql = qd.quad_list.cpu().numpy()
    for j, ent in enumerate(entries):
        assert ql[j * nb: j * nb + len(ent)].tolist() == ent
    assert qd.quad_stats.cpu().tolist() == [ptr[-1], int(mask.sum())]
    plan = fm.ForwardPlan(q.to(dev), k.to(dev), v.to(dev), lists, sm_scale,
                          out_dtype=torch.float32 if out_fp32 else None, quads=True)
    assert plan.uses_quads
    for _ in range(2):                       # the second run finds the counters as the first left them
        o, lse = plan.run()
        torch.cuda.synchronize()
        o_ref, lse_ref = orc.naive_attention(f32(q), f32(k), f32(v), mask.numpy(), sm_scale, return_lse=True)
        ma, rl = errors(o, o_ref)
        print("B%d H%d N%d %s fp32out=%s: max-abs %.3e rel-L2 %.3e" % (B, H, N, dtype, out_fp32, ma, rl))
        assert ma <= (2e-2 if dtype == torch.float16 else 3e-2)
        assert rl <= (1e-3 if dtype == torch.float16 or out_fp32 else 3e-3)
        fin = np.isfinite(lse_ref)
        l = lse.cpu().numpy()
        assert np.array_equal(np.isfinite(l), fin)
        assert np.abs(l[fin] - lse_ref[fin]).max() <= 2e-3
    return o


def test_dense_and_partial_last_quad(dev):
    run_case(dev, 1, 1, 256, torch.ones(1, 1, 4, 4, dtype=torch.bool))
    run_case(dev, 1, 1, 1088, torch.ones(1, 1, 17, 17, dtype=torch.bool), seed=1)     # 17 row blocks


def test_causal_and_random(dev):
    run_case(dev, 1, 1, 2048, causal_block_mask(1, 1, 32, 1.0, 0), seed=2)
    run_case(dev, 1, 1, 1024, uniform_block_mask(1, 1, 16, 0.5, 1), seed=3)
    run_case(dev, 1, 1, 4096, uniform_block_mask(1, 1, 64, 0.2, 2), seed=4)


def test_empty_rows(dev):
    g = torch.Generator().manual_seed(3)
    m = torch.rand(1, 1, 32, 32, generator=g) < 0.05            # no forced diagonal: some rows keep nothing
    assert bool((~m.any(-1)).any())
    o = run_case(dev, 1, 1, 2048, m, seed=5)
    empty = (~m[0, 0].any(-1)).nonzero().flatten().tolist()
    for r in empty:
        assert float(o[0, 0, 64 * r: 64 * r + 64].abs().max()) == 0.0


def test_heads_shared_and_own_masks(dev):
    run_case(dev, 2, 3, 1024, uniform_block_mask(1, 1, 16, 0.6, 4), seed=6)
    run_case(dev, 2, 3, 1024, uniform_block_mask(2, 3, 16, 0.6, 5), seed=7)
    run_case(dev, 1, 4, 4096, torch.ones(1, 1, 64, 64, dtype=torch.bool), seed=8)


def test_bf16(dev):
    run_case(dev, 1, 1, 1024, torch.ones(1, 1, 16, 16, dtype=torch.bool), dtype=torch.bfloat16, seed=9)
    run_case(dev, 1, 2, 1024, causal_block_mask(1, 1, 16, 1.0, 0), dtype=torch.bfloat16, seed=10, out_fp32=True)


def test_headline_shape_dense_rows_sampled(dev):
    """N=17536 dense: many ranges share every quad (the merge by the last arriver runs everywhere);
    checked on sampled row blocks against the oracle."""
    import fa2_custom_mask as fm
    N, nb = 17536, 274
    q, k, v = make_qkv(1, 1, N, 64, torch.float16, 11)
    mask = torch.ones(1, 1, nb, nb, dtype=torch.bool)
    lists = fm.block_mask_to_lists(mask.to(dev))
    plan = fm.ForwardPlan(q.to(dev), k.to(dev), v.to(dev), lists, 0.125, quads=True)
    o, lse = plan.run()
    torch.cuda.synchronize()
    for rb in (0, 1, 137, 272, 273):
        rows = slice(64 * rb, 64 * rb + 64)
        o_ref, lse_ref = orc.naive_attention(f32(q)[:, :, rows], f32(k), f32(v), mask.numpy()[:, :, rb:rb + 1], 0.125,
                                             return_lse=True)
        ma, rl = errors(o[:, :, rows], o_ref)
        assert ma <= 2e-2 and rl <= 1e-3
        assert np.abs(lse[:, :, rows].cpu().numpy() - lse_ref).max() <= 2e-3


def test_rejections(dev):
    import fa2_custom_mask as fm
    from fa2_custom_mask import _ext
    q, k, v = [x.to(dev) for x in make_qkv(1, 1, 256, 128, torch.float16, 0)]
    lists = fm.block_mask_to_lists(torch.ones(1, 1, 4, 4, dtype=torch.bool, device=dev))
    with pytest.raises(Exception):
        fm.ForwardPlan(q, k, v, lists, 0.1, quads=True).run()       # head dimension 128
    lib = _ext.lib()
    z = torch.zeros(16, dtype=torch.int32, device=dev)
    rc = lib.bsattn_quad_lists(z.data_ptr(), z.data_ptr(), 1, 1, 4096, z.data_ptr(), z.data_ptr(), z.data_ptr(), None)
    assert rc != 0                                                   # more row blocks than the kernel indexes
