"""GPU parity of the backward kernels against the CPU oracle's closed-form gradients
(algebra of fa2_bwd.py, pinned on the CPU against torch.autograd through the naive fp32 path).
Tolerances as the forward: max-abs 2e-2 (fp16) / 3e-2 (bf16); rel-L2 1e-3 on fp32-typed outputs
(bf16-typed outputs are limited by the output cast itself, 1.7e-3)."""
import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from helpers import make_qkv, uniform_block_mask, causal_block_mask, errors, f32, same_up_to_rounding

pytestmark = pytest.mark.gpu
MAXABS = {torch.float16: 2e-2, torch.bfloat16: 3e-2}


def run_case(dev, B, H, N, D, dtype, mask, seed, out_fp32):
    import fa2_custom_mask as fm
    q, k, v, do = make_qkv(B, H, N, D, dtype, seed, n=4)
    sc = 1.0 / np.sqrt(D)
    dq_r, dk_r, dv_r, _ = orc.attention_backward(f32(q), f32(k), f32(v), mask.numpy(), sc, f32(do))
    o_r, lse_r = orc.naive_attention(f32(q), f32(k), f32(v), mask.numpy(), sc, return_lse=True)
    o, lse, dq, dk, dv = fm.attention_forward_backward(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), sc,
                                                       do.to(dev), out_fp32=out_fp32)
    torch.cuda.synchronize()
    want = torch.float32 if out_fp32 else dtype
    for name, got, ref in (("O", o, o_r), ("dQ", dq, dq_r), ("dK", dk, dk_r), ("dV", dv, dv_r)):
        assert got.dtype == want and tuple(got.shape) == (B, H, N, D)
        ma, rl = errors(got, ref)
        print("%s B%d H%d N%d D%d %s fp32out=%s: max-abs %.3e rel-L2 %.3e" % (name, B, H, N, D, dtype, out_fp32, ma, rl))
        assert ma <= MAXABS[dtype]
        assert rl <= (1e-3 if (dtype == torch.float16 or out_fp32) else 3e-3)
    fin = np.isfinite(lse_r)
    assert np.abs(lse.cpu().numpy()[fin] - lse_r[fin]).max() <= 2e-3
    return dq, dk, dv


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128])
def test_small(dev, D, dtype):
    run_case(dev, 2, 2, 512, D, dtype, uniform_block_mask(2, 2, 8, 0.4, 3), 11, True)
    run_case(dev, 2, 2, 512, D, dtype, uniform_block_mask(2, 2, 8, 0.4, 3), 11, False)


def test_shared_causal_mask_c5_shape_small(dev):
    """C5's structure at reduced size: mask shared across heads, block-causal keep 0.25, bf16 D=128."""
    run_case(dev, 2, 4, 1024, 128, torch.bfloat16, causal_block_mask(1, 1, 16, 0.25, 5), 1238, True)


def test_empty_rows_and_columns(dev):
    m = uniform_block_mask(1, 2, 8, 0.3, 2)
    m[0, 0, 3, :] = False          # a query block without keys: dQ = 0 there
    m[0, 1, :, 5] = False          # a key block nobody attends to: dK = dV = 0 there
    dq, dk, dv = run_case(dev, 1, 2, 512, 64, torch.float16, m, 8, True)
    assert float(dq[0, 0, 192:256].abs().max()) == 0.0
    assert float(dk[0, 1, 320:384].abs().max()) == 0.0 and float(dv[0, 1, 320:384].abs().max()) == 0.0


def test_autograd_path(dev):
    """o.backward(do) through flash_attention_custom_mask, as the reference's users call it."""
    import fa2_custom_mask as fm
    B, H, N, D = 1, 2, 512, 64
    q, k, v, do = make_qkv(B, H, N, D, torch.float16, 21, n=4)
    mask = uniform_block_mask(1, 1, 8, 0.5, 21)
    sc = 0.125
    qd, kd, vd = [x.to(dev).requires_grad_(True) for x in (q, k, v)]
    o = fm.flash_attention_custom_mask(qd, kd, vd, mask.to(dev), sc)
    o.backward(do.to(dev))
    dq_r, dk_r, dv_r, _ = orc.attention_backward(f32(q), f32(k), f32(v), mask.numpy(), sc, f32(do))
    for got, ref in ((qd.grad, dq_r), (kd.grad, dk_r), (vd.grad, dv_r)):
        assert got.dtype == torch.float16
        ma, rl = errors(got, ref)
        assert ma <= 2e-2 and rl <= 1e-3
    # all-false mask: zeros forward (fa2_custom_mask.py:49-51) and zero gradients
    qd.grad = None
    z = fm.flash_attention_custom_mask(qd, kd, vd, torch.zeros(1, 1, 8, 8, dtype=torch.bool, device=dev), sc)
    z.backward(do.to(dev))
    assert float(z.abs().max()) == 0.0 and float(qd.grad.abs().max()) == 0.0


def test_invariant_rowsum_ds_zero(dev):
    """With dO = O-independent constant along d and v = const, dS rows sum to zero, so dQ = dK = 0."""
    import fa2_custom_mask as fm
    B, H, N, D = 1, 1, 1024, 64
    q, k, v, do = make_qkv(B, H, N, D, torch.float16, 4, n=4)
    mask = uniform_block_mask(1, 1, 16, 0.3, 4)
    vc = torch.ones_like(v) * 0.5
    _, _, dq, dk, dv = fm.attention_forward_backward(q.to(dev), k.to(dev), vc.to(dev), mask.to(dev), 0.125,
                                                     do.to(dev), out_fp32=True)
    assert float(dq.abs().max()) <= 2e-3 and float(dk.abs().max()) <= 2e-3


def test_strided_inputs_backward(dev):
    """q, k, v as views of one packed [B, N, 3, H, D] tensor (what a fused projection produces) and a
    strided dO: gradients equal those of contiguous copies up to the rounding of the forward's O (the
    forward hands tiles out dynamically, so two runs may round O differently; the backward itself has
    no atomics and is deterministic)."""
    import fa2_custom_mask as fm
    B, H, N, D = 2, 3, 256, 64
    g = torch.Generator().manual_seed(21)
    qkv = torch.randn(B, N, 3, H, D, generator=g).to(torch.float16).to(dev)
    q, k, v = [qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3)]
    do = torch.randn(B, N, H, D, generator=g).to(torch.float16).to(dev).permute(0, 2, 1, 3)
    m = uniform_block_mask(1, 1, N // 64, 0.6, 22).to(dev)
    res_s = fm.attention_forward_backward(q, k, v, m, 0.125, do)
    res_c = fm.attention_forward_backward(q.contiguous(), k.contiguous(), v.contiguous(), m, 0.125, do.contiguous())
    from helpers import same_up_to_rounding
    for a, b_ in zip(res_s[2:], res_c[2:]):
        assert same_up_to_rounding(a, b_, rel=2.0 ** -8, abs_=2e-3)


def test_backward_plan_matches_the_call(dev):
    """BackwardPlan (buffers and arguments prepared once) against attention_forward_backward, run
    twice on a workspace filled with ones in between (split lists: fp32 parts in the workspace)."""
    import fa2_custom_mask as fm
    B, H, N, D = 1, 2, 2048, 128
    q, k, v, do = [x.to(dev) for x in make_qkv(B, H, N, D, torch.bfloat16, 611, n=4)]
    mask = causal_block_mask(1, 1, N // 64, 0.5, 612).to(dev)
    sc = 1.0 / np.sqrt(D)
    o, lse, dq, dk, dv = fm.attention_forward_backward(q, k, v, mask, sc, do)
    lists = fm.block_mask_to_lists(mask)
    lists_t = fm.block_mask_to_lists(mask, transpose=True)
    plan = fm.BackwardPlan(q, k, v, o, do, lse, lists, lists_t, sc)
    for fill in (None, 255):
        if fill is not None:
            plan.ws.fill_(fill)
        for t in (plan.dq, plan.dk, plan.dv):
            t.fill_(float("nan"))
        got = plan.run()
        torch.cuda.synchronize()
        for a, b_ in zip(got, (dq, dk, dv)):
            assert same_up_to_rounding(a, b_, rel=2.0 ** -8, abs_=2e-3)
    with pytest.raises(ValueError):
        fm.BackwardPlan(q[:, :, :100], k[:, :, :100], v[:, :, :100], o[:, :, :100], do[:, :, :100], lse[:, :, :100],
                        lists, lists_t, sc)


@pytest.mark.parametrize("out_fp32", [False, True])
def test_packed_qkv_layout_is_kept(dev, out_fp32):
    """q, k, v sliced out of one packed [B, N, 3, H, D] tensor (no copies): o, dq, dk, dv come back in the
    layout torch.empty_like gives for such inputs, which is what the reference allocates
    (fa2_custom_mask.py:59, 101-103), and the kernels write through those strides."""
    import fa2_custom_mask as fm
    B, H, N, D = 2, 3, 512, 64
    g = torch.Generator().manual_seed(41)
    qkv = torch.randn(B, N, 3, H, D, generator=g).to(torch.float16)
    do = torch.randn(B, N, H, D, generator=g).to(torch.float16)
    mask = uniform_block_mask(1, 3, 8, 0.4, 9)
    sc = 0.125
    qkv_d, do_d = qkv.to(dev), do.to(dev)
    q, k, v = [qkv_d[:, :, i].transpose(1, 2) for i in range(3)]          # [B, H, N, D] views
    assert not q.is_contiguous()
    o, lse, dq, dk, dv = fm.attention_forward_backward(q, k, v, mask.to(dev), sc, do_d.transpose(1, 2), out_fp32=out_fp32)
    torch.cuda.synchronize()
    want = torch.empty_like(q, dtype=torch.float32 if out_fp32 else torch.float16).stride()
    assert want == (N * H * D, D, H * D, 1)
    for t in (o, dq, dk, dv):
        assert t.stride() == want
    qc, kc, vc = [f32(qkv[:, :, i].transpose(1, 2).contiguous()) for i in range(3)]
    doc = f32(do.transpose(1, 2).contiguous())
    dq_r, dk_r, dv_r, _ = orc.attention_backward(qc, kc, vc, mask.numpy(), sc, doc)
    o_r = orc.naive_attention(qc, kc, vc, mask.numpy(), sc)
    for got, ref in ((o, o_r), (dq, dq_r), (dk, dk_r), (dv, dv_r)):
        ma, rl = errors(got, ref)
        assert ma <= 2e-2 and rl <= 1e-3


@pytest.mark.parametrize("out_fp32", [False, True])
def test_packed_qkv_layout_d128_whole_lists(dev, out_fp32):
    """Packed [B, N, 3, H, D] inputs at D = 128 with enough row blocks that every list belongs to one workgroup: the
    pair forward kernel, dq_kernel and dkdv4_kernel then write their result rows themselves, through LDS and through
    the strides of the results.  Two heads against the oracle, all heads against the same call on contiguous copies."""
    import fa2_custom_mask as fm
    B, H, N, D, nb = 2, 8, 4096, 128, 64
    g = torch.Generator().manual_seed(43)
    qkv = torch.randn(B, N, 3, H, D, generator=g).to(torch.bfloat16)
    do = torch.randn(B, N, H, D, generator=g).to(torch.bfloat16)
    mask = uniform_block_mask(1, 1, nb, 0.3, 11)
    sc = 1.0 / np.sqrt(D)
    qkv_d, do_d = qkv.to(dev), do.to(dev)
    q, k, v = [qkv_d[:, :, i].transpose(1, 2) for i in range(3)]
    res = fm.attention_forward_backward(q, k, v, mask.to(dev), sc, do_d.transpose(1, 2), out_fp32=out_fp32)
    want = torch.empty_like(q, dtype=torch.float32 if out_fp32 else torch.bfloat16).stride()
    for t in (res[0], res[2], res[3], res[4]):
        assert t.stride() == want == (N * H * D, D, H * D, 1)
    ref = fm.attention_forward_backward(q.contiguous(), k.contiguous(), v.contiguous(), mask.to(dev), sc,
                                        do_d.transpose(1, 2).contiguous(), out_fp32=out_fp32)
    for a_, b_ in zip(res, ref):
        assert torch.equal(a_, b_)                        # the layout of the results changes no value
    for (b, h) in ((0, 1), (1, 6)):
        qh, kh, vh = [f32(qkv[b:b + 1, :, i, h:h + 1].transpose(1, 2).contiguous()) for i in range(3)]
        doh = f32(do[b:b + 1, :, h:h + 1].transpose(1, 2).contiguous())
        o_r = orc.naive_attention(qh, kh, vh, mask.numpy(), sc)
        dq_r, dk_r, dv_r, _ = orc.attention_backward(qh, kh, vh, mask.numpy(), sc, doh)
        for got, r in ((res[0], o_r), (res[2], dq_r), (res[3], dk_r), (res[4], dv_r)):
            ma, rl = errors(got[b:b + 1, h:h + 1], r)
            assert ma <= 3e-2 and rl <= (1e-3 if out_fp32 else 3e-3)


def test_packed_qkv_split_lists(dev):
    """The same for a single long head, whose row and column lists are walked by several workgroups (the
    gradients are then summed from fp32 parts by a kernel of its own, which writes through the strides)."""
    import fa2_custom_mask as fm
    B, H, N, D = 1, 1, 2048, 64
    g = torch.Generator().manual_seed(42)
    qkv = torch.randn(B, N, 3, H, D, generator=g).to(torch.float16)
    do = torch.randn(B, H, N, D, generator=g).to(torch.float16)
    mask = uniform_block_mask(1, 1, 32, 0.5, 10)
    qkv_d = qkv.to(dev)
    q, k, v = [qkv_d[:, :, i].transpose(1, 2) for i in range(3)]
    o, lse, dq, dk, dv = fm.attention_forward_backward(q, k, v, mask.to(dev), 0.125, do.to(dev))
    torch.cuda.synchronize()
    qc, kc, vc = [f32(qkv[:, :, i].transpose(1, 2).contiguous()) for i in range(3)]
    dq_r, dk_r, dv_r, _ = orc.attention_backward(qc, kc, vc, mask.numpy(), 0.125, f32(do))
    for got, ref in ((dq, dq_r), (dk, dk_r), (dv, dv_r)):
        assert got.stride() == torch.empty_like(q).stride()
        ma, rl = errors(got, ref)
        assert ma <= 2e-2 and rl <= 1e-3


def test_delta_against_oracle(dev):
    """delta = rowsum(O * dO) (fa2_bwd.py:17), the first step of the backward, lives at the start of the
    workspace: compared with the oracle's directly, not only through the gradients."""
    import fa2_custom_mask as fm
    B, H, N, D = 2, 2, 1024, 128
    q, k, v, do = make_qkv(B, H, N, D, torch.float16, 43, n=4)
    mask = uniform_block_mask(1, 1, 16, 0.4, 11)
    sc = 1.0 / np.sqrt(D)
    lists = fm.block_mask_to_lists(mask.to(dev))
    lists_t = fm.block_mask_to_lists(mask.to(dev), transpose=True)
    qd, kd, vd, dod = [x.to(dev) for x in (q, k, v, do)]
    o, lse = fm.ForwardPlan(qd, kd, vd, lists, sc).run()
    plan = fm.BackwardPlan(qd, kd, vd, o, dod, lse, lists, lists_t, sc)
    plan.run()
    torch.cuda.synchronize()
    delta = plan.ws[:B * H * N * 4].view(torch.float32).reshape(B, H, N).cpu().numpy()
    _, _, _, delta_r = orc.attention_backward(f32(q), f32(k), f32(v), mask.numpy(), sc, f32(do))
    # O enters as the fp16-rounded forward result: 2^-11 relative per term, D terms of random sign
    assert np.abs(delta - delta_r).max() <= 5e-3
    assert np.linalg.norm(delta - delta_r) / np.linalg.norm(delta_r) <= 2e-3


def test_large_magnitudes_backward_d128_fp16(dev):
    """fp16 inputs at D = 128 whose per-query terms lie above fp16's range: raw scores q k^T of the order of 1e5
    (so lse / sm_scale does too) and delta = rowsum(O dO) above 1e5 (values with a large common component, as
    gradients under loss scaling meet them), while P and dS = P (dP - delta) themselves stay representable (the
    reference rounds both to fp16 as well, fa2_bwd.py:66,73,127).  The dK/dV kernel feeds lse and delta through a
    contraction slice as 16-bit pieces: they must not overflow.  With delta this large against dP - delta the
    rounding of the stored O matters (1 % of dQ and dK here): the oracle takes delta from the same fp16 O the
    kernels are given, as the reference does (fa2_bwd.py:15-17)."""
    import fa2_custom_mask as fm
    B, H, N, D = 1, 2, 512, 128
    g = torch.Generator().manual_seed(91)
    q = (torch.randn(B, H, N, D, generator=g) * 40.0).to(torch.float16)
    k = (torch.randn(B, H, N, D, generator=g) * 40.0).to(torch.float16)
    v0 = 300.0 * torch.sign(torch.randn(1, H, 1, D, generator=g))
    v = (v0 + 20.0 * torch.randn(B, H, N, D, generator=g)).to(torch.float16)
    do = (torch.randn(B, H, N, D, generator=g) * 30.0).to(torch.float16)
    mask = uniform_block_mask(1, 1, 8, 0.5, 13)
    sc = 0.001
    o_r, lse_r = orc.naive_attention(f32(q), f32(k), f32(v), mask.numpy(), sc, return_lse=True)
    o, lse, dq, dk, dv = fm.attention_forward_backward(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), sc, do.to(dev),
                                                       out_fp32=True)
    torch.cuda.synchronize()
    assert errors(o, o_r)[1] <= 2e-3
    o16 = o.to(torch.float16)                   # what attention_forward_backward hands to the backward
    dq_r, dk_r, dv_r, delta_r = orc.attention_backward(f32(q), f32(k), f32(v), mask.numpy(), sc, f32(do),
                                                       dtype=np.float64, o_stored=f32(o16))
    assert np.abs(delta_r).max() > 65504.0 and np.abs(lse_r).max() / sc > 65504.0     # the case this test is for
    for name, got, ref in (("dQ", dq, dq_r), ("dK", dk, dk_r), ("dV", dv, dv_r)):
        assert bool(torch.isfinite(got).all()), name
        ma, rl = errors(got, ref)
        print("%s: max-abs %.3e of %.3e, rel-L2 %.3e" % (name, ma, float(np.abs(ref).max()), rl))
        # (the softmax is nearly one-hot and the exponents carry the rounding of the 16-bit scaled Q: a looser
        # bar than for N(0,1) data; an overflowing piece gives NaN or errors of the size of the result)
        assert rl <= 5e-3, name
