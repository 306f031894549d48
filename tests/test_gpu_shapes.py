"""Shapes the reference advertises but does not run (fa2_custom_mask.py:43,58; fa2_fwd.py:120):
sequence lengths that are not a multiple of 64 and head dimensions 16 and 32.  Checked against the
CPU oracle's naive masked softmax (kernel-test.py:37-40) on the mask expanded as kernel-test.py:18
and cut to N x N, and against its backward."""
import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from helpers import make_qkv, errors, f32, uniform_block_mask

pytestmark = pytest.mark.gpu

MAXABS = {torch.float16: 2e-2, torch.bfloat16: 3e-2}


def cut_mask(block, N):
    """Block mask [.., nb, nb] -> elementwise [.., N, N]: expanded (kernel-test.py:18), then cut."""
    return orc.expand_block_mask(block.numpy())[..., :N, :N]


def check(dev, B, H, N, D, dtype, mask_dev_form, mask_oracle, seed, backward=True):
    import fa2_custom_mask as fm
    q, k, v, do = make_qkv(B, H, N, D, dtype, seed, n=4)
    sc = 1.0 / np.sqrt(D)
    o_ref, lse_ref = orc.naive_attention(f32(q), f32(k), f32(v), mask_oracle, sc, return_lse=True)
    m = None if mask_dev_form is None else mask_dev_form.to(dev)
    o, lse, dq, dk, dv = fm.attention_forward_backward(q.to(dev), k.to(dev), v.to(dev), m, sc, do.to(dev), out_fp32=True)
    torch.cuda.synchronize()
    assert o.shape == (B, H, N, D) and lse.shape == (B, H, N) and dq.shape == dk.shape == dv.shape == (B, H, N, D)
    ma, rl = errors(o, o_ref)
    print("B%d H%d N%d D%d %s: O max-abs %.3e rel-L2 %.3e" % (B, H, N, D, dtype, ma, rl))
    assert ma <= MAXABS[dtype] and rl <= 1e-3
    fin = np.isfinite(lse_ref)
    assert np.array_equal(np.isfinite(lse.cpu().numpy()), fin)
    assert np.abs(lse.cpu().numpy()[fin] - lse_ref[fin]).max() <= 2e-3
    if backward:
        refs = orc.attention_backward(f32(q), f32(k), f32(v), mask_oracle, sc, f32(do))
        for name, x, r in zip(("dq", "dk", "dv"), (dq, dk, dv), refs):
            ma, rl = errors(x, r)
            print("   %s max-abs %.3e rel-L2 %.3e" % (name, ma, rl))
            assert ma <= MAXABS[dtype] and (rl <= 1e-3 or ma <= 1e-5), name   # (a zero gradient has no relative error)
    return o


@pytest.mark.parametrize("N", [1, 50, 64, 65, 200, 777])
@pytest.mark.parametrize("D,dtype", [(64, torch.float16), (128, torch.bfloat16)])
def test_ragged_length_block_mask(dev, N, D, dtype):
    nb = -(-N // 64)
    block = uniform_block_mask(1, 2, nb, 0.6, 70 + N)
    check(dev, 1, 2, N, D, dtype, block, cut_mask(block, N), 71 + N)


@pytest.mark.parametrize("N", [100, 333])
def test_ragged_length_elementwise_mask_and_none(dev, N):
    g = torch.Generator().manual_seed(72)
    m = torch.rand(2, 1, N, N, generator=g) < 0.4
    m[0, 0, 7, :] = False                          # a query without keys
    check(dev, 2, 3, N, 64, torch.float16, m, m.numpy(), 73)
    check(dev, 1, 2, N, 64, torch.float16, None, np.ones((1, 1, N, N), dtype=bool), 74)


def test_ragged_length_autograd(dev):
    """The autograd entry returns gradients of the callers' shapes."""
    import fa2_custom_mask as fm
    N, D = 150, 64
    q, k, v, do = [x.to(dev) for x in make_qkv(1, 2, N, D, torch.float16, 75, n=4)]
    block = uniform_block_mask(1, 1, 3, 0.7, 76)
    q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)
    o = fm.flash_attention_custom_mask(q, k, v, block.to(dev), 0.125)
    assert o.shape == (1, 2, N, D)
    o.backward(do)
    refs = orc.attention_backward(f32(q), f32(k), f32(v), cut_mask(block, N), 0.125, f32(do))
    for x, r in zip((q.grad, k.grad, v.grad), refs):
        assert x.shape == (1, 2, N, D)
        ma, rl = errors(x, r)
        assert ma <= 2e-2 and rl <= 2e-3          # gradients come back rounded to fp16


@pytest.mark.parametrize("D", [16, 32])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_small_head_dims(dev, D, dtype):
    block = uniform_block_mask(1, 1, 4, 0.5, 77)
    check(dev, 2, 2, 256, D, dtype, block, cut_mask(block, 256), 78 + D)
    check(dev, 1, 1, 90, D, dtype, None, np.ones((1, 1, 90, 90), dtype=bool), 79 + D)


def test_tail_words_bit_exact(dev):
    """bsattn_tail_mask_tiles against the oracle's packing of the cut mask padded with False."""
    import fa2_custom_mask as fm
    from fa2_custom_mask import utils
    N, nb = 150, 3
    block = uniform_block_mask(2, 1, nb, 0.6, 80)
    dense = np.zeros((2, 1, nb * 64, nb * 64), dtype=bool)
    dense[..., :N, :] = orc.expand_block_mask(block.numpy())[..., :N, :]
    dense[..., N:] = False                                  # padding keys
    dense[..., N:, :N] = orc.expand_block_mask(block.numpy())[..., N:, :N]   # padding queries keep their block's keys
    for tr in (False, True):
        lists = fm.block_mask_to_lists(block.to(dev), transpose=tr)
        partial, bits = utils.tail_mask_tiles(lists, N - 128, transpose=tr)
        T = int(lists.counts[1])
        p_ref, w_ref = orc.pack_mask_tiles(dense, transpose=tr)
        assert np.array_equal(partial[:T].cpu().numpy(), p_ref)
        assert np.array_equal(bits[:T].cpu().numpy().view(np.uint64), w_ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_head_dim_256(dev, dtype):
    """D = 256 (fa2_custom_mask.py:58 lists it): forward, LSE and gradients against the oracle, block mask, elementwise
    mask with partly set tiles and queries without keys, a sequence length that is not a multiple of 64, and a
    launch with few row blocks (row and column lists shared between workgroups in the backward)."""
    block = uniform_block_mask(1, 2, 8, 0.5, 90)
    block[0, 0, 3, :] = False
    check(dev, 1, 2, 512, 256, dtype, block, cut_mask(block, 512), 91)
    g = torch.Generator().manual_seed(92)
    m = (torch.rand(1, 1, 200, 200, generator=g) < 0.4) & torch.tril(torch.ones(200, 200, dtype=torch.bool))
    m[0, 0, 9, :] = False
    check(dev, 2, 3, 200, 256, dtype, m, m.numpy(), 93)
    long_block = uniform_block_mask(1, 1, 32, 0.6, 94)
    check(dev, 1, 1, 2048, 256, dtype, long_block, cut_mask(long_block, 2048), 95)


def test_head_dim_256_bf16_typed_results_many_heads(dev):
    import fa2_custom_mask as fm
    B, H, N, D = 2, 32, 256, 256
    q, k, v, do = make_qkv(B, H, N, D, torch.bfloat16, 96, n=4)
    block = uniform_block_mask(1, 1, 4, 0.7, 97)
    sc = 1.0 / 16.0
    o, lse, dq, dk, dv = fm.attention_forward_backward(q.to(dev), k.to(dev), v.to(dev), block.to(dev), sc, do.to(dev))
    torch.cuda.synchronize()
    for hd in (0, 63):
        b, h = divmod(hd, H)
        sl = (slice(b, b + 1), slice(h, h + 1))
        o_ref = orc.naive_attention(f32(q[sl]), f32(k[sl]), f32(v[sl]), cut_mask(block, N), sc)
        refs = orc.attention_backward(f32(q[sl]), f32(k[sl]), f32(v[sl]), cut_mask(block, N), sc, f32(do[sl]))
        for got, ref in ((o, o_ref), (dq, refs[0]), (dk, refs[1]), (dv, refs[2])):
            assert got.dtype == torch.bfloat16
            ma, rl = errors(got[sl], ref)
            assert ma <= 3e-2 and rl <= 4e-3


def test_unsupported_head_dim_is_an_error(dev):
    import fa2_custom_mask as fm
    q = torch.zeros(1, 1, 128, 512, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        fm.flash_attention_custom_mask(q, q, q, None, 0.1)
    q = torch.zeros(1, 1, 128, 48, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        fm.flash_attention_custom_mask(q, q, q, None, 0.1)
