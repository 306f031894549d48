"""GPU parity of the elementwise-mask path (exact semantics inside partly set tiles) against the
CPU oracle's naive masked softmax (kernel-test.py:37-40 with the mask used as it is)."""
import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from helpers import make_qkv, errors, f32

pytestmark = pytest.mark.gpu

MAXABS = {torch.float16: 2e-2, torch.bfloat16: 3e-2}


def token_causal(N):
    return torch.tril(torch.ones(N, N, dtype=torch.bool)).reshape(1, 1, N, N)


def check_forward(dev, B, H, N, D, dtype, mask, seed, q_gain=1.0):
    import fa2_custom_mask as fm
    q, k, v = make_qkv(B, H, N, D, dtype, seed)
    q = (q.float() * q_gain).to(dtype)
    sc = 1.0 / np.sqrt(D)
    o_ref, lse_ref = orc.naive_attention(f32(q), f32(k), f32(v), mask.numpy(), sc, return_lse=True)
    o, lse = fm.flash_attention_custom_mask_lse(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), sc, out_fp32=True)
    torch.cuda.synchronize()
    ma, rl = errors(o, o_ref)
    print("B%d H%d N%d D%d %s gain %.0f: max-abs %.3e rel-L2 %.3e" % (B, H, N, D, dtype, q_gain, ma, rl))
    assert ma <= MAXABS[dtype] and rl <= 1e-3
    fin = np.isfinite(lse_ref)
    l = lse.cpu().numpy()
    assert np.array_equal(np.isfinite(l), fin)
    assert np.abs(l[fin] - lse_ref[fin]).max() <= 2e-3 * max(1.0, q_gain)
    assert float(np.abs(f32(o)[~fin]).max() if (~fin).any() else 0.0) == 0.0
    return o


@pytest.mark.parametrize("D,dtype", [(64, torch.float16), (128, torch.bfloat16), (64, torch.bfloat16), (128, torch.float16)])
def test_token_causal_mask(dev, D, dtype):
    """Token-level causal mask: every diagonal tile is partly set, tiles below are full."""
    check_forward(dev, 1, 2, 512, D, dtype, token_causal(512), 51)


@pytest.mark.parametrize("D,dtype", [(64, torch.float16), (128, torch.bfloat16)])
def test_random_elementwise_masks(dev, D, dtype):
    g = torch.Generator().manual_seed(52)
    N = 512
    m = torch.rand(2, 3, N, N, generator=g) < 0.5
    m[0, 0, :, 64:128] = False                 # empty tiles
    m[0, 1, 128:256, :] = True                 # full tiles
    m[1, 2, 200:210, :] = False                # queries without any key
    m[1, 0, :64, :] = False                    # a whole row block without keys
    m[1, 1, 5, :] = False
    m[1, 1, 5, 300] = True                     # one key only
    check_forward(dev, 2, 3, N, D, dtype, m, 53)
    check_forward(dev, 2, 3, N, D, dtype, m[:1, :1], 54)          # shared by all heads


def test_first_tiles_masked_and_large_scores(dev):
    """Queries whose first kept tiles are masked for them start without a reference exponent; with
    large negative or positive scores afterwards nothing may underflow or overflow."""
    g = torch.Generator().manual_seed(55)
    N = 1024
    m = torch.zeros(1, 1, N, N, dtype=torch.bool)
    m[0, 0] = torch.rand(N, N, generator=g) < 0.3
    m[0, 0, ::2, :448] = False                 # even queries: nothing in the first seven tiles
    m[0, 0, 0, :] = False
    m[0, 0, 0, N - 1] = True
    for gain in (1.0, 8.0):
        check_forward(dev, 1, 1, N, 64, torch.float16, m, 56, q_gain=gain)


def test_many_heads_elementwise(dev):
    """Row-block-per-wavefront mode (many heads) with partly set tiles."""
    g = torch.Generator().manual_seed(57)
    N = 512
    m = (torch.rand(1, 1, N, N, generator=g) < 0.6) & token_causal(N)
    m[0, 0, 70, :] = False
    check_forward(dev, 4, 64, N, 64, torch.float16, m, 58)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_many_heads_elementwise_d128(dev, dtype):
    """D = 128 with many row blocks in the launch (one wavefront pair per row block) and partly set
    tiles, queries without keys, an empty row block."""
    g = torch.Generator().manual_seed(64)
    N = 512
    m = (torch.rand(1, 1, N, N, generator=g) < 0.6) & token_causal(N)
    m[0, 0, 70, :] = False
    m[0, 0, 128:192, :] = False
    check_forward(dev, 4, 64, N, 128, dtype, m, 65)
    m2 = torch.rand(4, 1, N, N, generator=g) < 0.3
    m2[2, 0, :, :64] = False
    check_forward(dev, 4, 64, N, 128, dtype, m2, 66)


def test_tile_constant_elementwise_equals_block(dev):
    import fa2_custom_mask as fm
    from helpers import uniform_block_mask, same_up_to_rounding
    N = 1024
    block = uniform_block_mask(1, 2, N // 64, 0.4, 59)
    dense = block.repeat_interleave(64, 2).repeat_interleave(64, 3)
    q, k, v = [x.to(dev) for x in make_qkv(1, 2, N, 64, torch.float16, 60)]
    assert same_up_to_rounding(fm.flash_attention_custom_mask(q, k, v, dense.to(dev), 0.125),
                               fm.flash_attention_custom_mask(q, k, v, block.to(dev), 0.125))


@pytest.mark.parametrize("D,dtype", [(64, torch.float16), (128, torch.bfloat16), (128, torch.float16)])
def test_backward_elementwise(dev, D, dtype):
    """dQ, dK, dV with elementwise masks (token-causal, and random with empty tiles, full tiles and
    queries without keys) against the oracle's gradient of the naive masked softmax."""
    import fa2_custom_mask as fm
    g = torch.Generator().manual_seed(61)
    N = 384
    rnd = torch.rand(1, 2, N, N, generator=g) < 0.4
    rnd[0, 0, :, 64:128] = False
    rnd[0, 1, 128:192, :] = True
    rnd[0, 1, 7, :] = False
    rnd[0, 0, 320:, :] = False
    for mask in (token_causal(N), rnd):
        H = 2
        q, k, v, do = make_qkv(1, H, N, D, dtype, 62, n=4)
        sc = 1.0 / np.sqrt(D)
        dq_r, dk_r, dv_r, _ = orc.attention_backward(f32(q), f32(k), f32(v), mask.numpy(), sc, f32(do))
        o, lse, dq, dk, dv = fm.attention_forward_backward(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), sc,
                                                           do.to(dev), out_fp32=True)
        torch.cuda.synchronize()
        for name, got, ref in (("dq", dq, dq_r), ("dk", dk, dk_r), ("dv", dv, dv_r)):
            ma, rl = errors(got, ref)
            print("%s D%d %s: max-abs %.3e rel-L2 %.3e" % (name, D, dtype, ma, rl))
            assert np.isfinite(f32(got)).all()
            assert ma <= MAXABS[dtype] and rl <= 1e-3


def test_autograd_with_elementwise_mask(dev):
    import fa2_custom_mask as fm
    N = 256
    mask = token_causal(N)
    q, k, v, do = make_qkv(1, 1, N, 64, torch.float16, 63, n=4)
    dq_r, dk_r, dv_r, _ = orc.attention_backward(f32(q), f32(k), f32(v), mask.numpy(), 0.125, f32(do))
    qd, kd, vd = [x.to(dev).requires_grad_(True) for x in (q, k, v)]
    fm.flash_attention_custom_mask(qd, kd, vd, mask.to(dev), 0.125).backward(do.to(dev))
    for got, ref in ((qd.grad, dq_r), (kd.grad, dk_r), (vd.grad, dv_r)):
        assert errors(got, ref)[0] <= 2e-2


@pytest.mark.parametrize("D,B,H", [(64, 1, 2), (128, 1, 2), (128, 4, 64)])
def test_bf16_typed_outputs_elementwise(dev, D, B, H):
    """bf16 inputs with bf16-typed results (P and dS rounded to bf16, no tile converted): forward and
    gradients with an elementwise mask against the oracle; the cast of an exact result to bf16 alone is
    1.7e-3 in rel-L2, hence the 3e-3 bar.  (B, H) = (4, 64) takes the many-row-blocks forward at D = 128."""
    import fa2_custom_mask as fm
    g = torch.Generator().manual_seed(67)
    N = 384
    mask = (torch.rand(1, 1, N, N, generator=g) < 0.5) & token_causal(N)
    mask[0, 0, 100, :] = False
    q, k, v, do = make_qkv(B, H, N, D, torch.bfloat16, 68, n=4)
    sc = 1.0 / np.sqrt(D)
    hs = slice(0, 2)                                   # oracle on two heads of the first batch entry
    o_r = orc.naive_attention(f32(q[:1, hs]), f32(k[:1, hs]), f32(v[:1, hs]), mask.numpy(), sc)
    dq_r, dk_r, dv_r, _ = orc.attention_backward(f32(q[:1, hs]), f32(k[:1, hs]), f32(v[:1, hs]), mask.numpy(), sc,
                                                 f32(do[:1, hs]))
    o, lse, dq, dk, dv = fm.attention_forward_backward(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), sc, do.to(dev))
    torch.cuda.synchronize()
    for name, got, ref in (("o", o, o_r), ("dq", dq, dq_r), ("dk", dk, dk_r), ("dv", dv, dv_r)):
        assert got.dtype == torch.bfloat16
        ma, rl = errors(got[:1, hs], ref)
        print("%s D%d: max-abs %.3e rel-L2 %.3e" % (name, D, ma, rl))
        assert ma <= 3e-2 and rl <= 3e-3, name


def test_large_scores_with_half_masked_queries_many_heads(dev):
    """A query's 64 keys of a tile sit in two lanes.  With large score differences one lane's share of P can
    round to zero while the other lane holds all the mass: both must still follow one reference
    exponent.  Many heads, so that a wavefront walks whole row blocks (several tiles in a row)."""
    g = torch.Generator().manual_seed(69)
    N = 1024
    m = torch.rand(1, 1, N, N, generator=g) < 0.3
    m[0, 0, ::2, :448] = False
    q, k, v = make_qkv(1, 1, N, 64, torch.float16, 70)
    q = (q.float() * 8.0).to(torch.float16)
    o_ref, lse_ref = orc.naive_attention(f32(q), f32(k), f32(v), m.numpy(), 0.125, return_lse=True)
    import fa2_custom_mask as fm
    H = 256
    qq, kk, vv = [x.expand(1, H, N, 64).contiguous().to(dev) for x in (q, k, v)]
    o, lse = fm.flash_attention_custom_mask_lse(qq, kk, vv, m.to(dev), 0.125, out_fp32=True)
    torch.cuda.synchronize()
    for hd in (0, 100, 255):
        ma, rl = errors(o[:, hd:hd + 1], o_ref)
        assert ma <= 2e-2 and rl <= 1e-3
        assert np.abs(lse[:, hd:hd + 1].cpu().numpy() - lse_ref).max() <= 2e-2
