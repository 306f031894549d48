"""The hand-off between workgroups that share a row block (the kernels behind bsattn_fwd): nobody waits, the
workgroup that counts itself in last merges the parts in the order of the ranges.  Checked where it
matters: with the deterministic switch two runs give the same bits, and a launch that is confined to a few
compute units from the host (so that most workgroups of a row block are never resident together) gives the
same bits again."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from helpers import make_qkv, uniform_block_mask, errors, f32

pytestmark = pytest.mark.gpu


@pytest.fixture
def deterministic():
    import fa2_custom_mask as fm
    before = fm.set_deterministic(True)
    yield
    fm.set_deterministic(before)


CASES = [
    # B, H, N, D, keep (1.0: dense), dtype
    (1, 1, 17536, 64, 1.0, torch.float16),      # every row block is shared by about two workgroups
    (1, 1, 17536, 64, 0.1, torch.float16),
    (1, 2, 4096, 64, 0.5, torch.bfloat16),
    (1, 1, 8192, 128, 0.5, torch.float16),
    (1, 1, 2048, 256, 1.0, torch.float16),      # row lists shared by the kernel for head dimension 256
]


def _plan(dev, B, H, N, D, keep, dtype, stream=None, seed=5):
    import fa2_custom_mask as fm
    q, k, v = [x.to(dev) for x in make_qkv(B, H, N, D, dtype, seed)]
    nb = N // 64
    mask = torch.ones(1, 1, nb, nb, dtype=torch.bool) if keep >= 1.0 else uniform_block_mask(1, 1, nb, keep, seed)
    lists = fm.block_mask_to_lists(mask.to(dev))
    torch.cuda.synchronize()
    return fm.ForwardPlan(q, k, v, lists, 1.0 / np.sqrt(D), stream=stream), mask


@pytest.mark.parametrize("case", CASES)
def test_two_runs_give_the_same_bits(dev, deterministic, case):
    plan, _ = _plan(dev, *case)
    o1, l1 = [t.clone() for t in plan.run()]
    torch.cuda.synchronize()
    for _ in range(3):
        o2, l2 = plan.run()
        torch.cuda.synchronize()
        assert torch.equal(o1.view(torch.int16), o2.view(torch.int16))
        assert torch.equal(l1.view(torch.int32), l2.view(torch.int32))


def _masked_stream(n_cus):
    """A stream whose kernels run on the first n_cus compute units only (hipExtStreamCreateWithCUMask)."""
    hip = ctypes.CDLL("libamdhip64.so")
    words = (ctypes.c_uint32 * 8)()
    for i in range(n_cus):
        words[i // 32] |= 1 << (i % 32)
    handle = ctypes.c_void_p()
    try:
        rc = hip.hipExtStreamCreateWithCUMask(ctypes.byref(handle), 8, words)
    except AttributeError:
        pytest.skip("this HIP runtime has no hipExtStreamCreateWithCUMask")
    if rc != 0 or not handle.value:
        pytest.skip("hipExtStreamCreateWithCUMask failed with %d" % rc)
    return hip, handle


@pytest.mark.parametrize("case", CASES[:1] + CASES[3:4])
def test_few_resident_workgroups_give_the_same_bits(dev, deterministic, case):
    """At most 16 (D = 64) or 8 (D = 128) of the launch's workgroups run at a time: the holders of a
    row block's parts rarely overlap in time, and the last of them still finds every part."""
    B, H, N, D, keep, dtype = case
    plan, mask = _plan(dev, *case)
    o_all, lse_all = [t.clone() for t in plan.run()]
    torch.cuda.synchronize()
    hip, handle = _masked_stream(8)
    try:
        narrow, _ = _plan(dev, *case, stream=torch.cuda.ExternalStream(handle.value))
        o, lse = narrow.run()
        assert hip.hipStreamSynchronize(handle) == 0
        torch.cuda.synchronize()
        assert torch.equal(o_all.view(torch.int16), o.view(torch.int16))
        assert torch.equal(lse_all.view(torch.int32), lse.view(torch.int32))
    finally:
        hip.hipStreamDestroy(handle)
    # and the bits are right: sampled row blocks against the oracle
    q, k, v = make_qkv(B, H, N, D, dtype, 5)
    for rb in (0, N // 128, N // 64 - 1):
        rows = slice(64 * rb, 64 * rb + 64)
        o_ref, _ = orc.naive_attention(f32(q)[:, :, rows], f32(k), f32(v), mask.numpy()[:, :, rb:rb + 1],
                                       1.0 / np.sqrt(D), return_lse=True)
        ma, rl = errors(o[:, :, rows], o_ref)
        assert ma <= 2e-2 and rl <= 1e-3


def test_default_mode_agrees_up_to_rounding(dev):
    """Without the switch the order of summation inside a workgroup follows the pace of its wavefronts:
    the same values up to the rounding of the 16-bit result."""
    from helpers import same_up_to_rounding
    import fa2_custom_mask as fm
    assert fm.set_deterministic(False) is False
    plan, _ = _plan(dev, 1, 1, 17536, 64, 1.0, torch.float16)
    o1 = plan.run()[0].clone()
    fm.set_deterministic(True)
    try:
        o2 = plan.run()[0].clone()
    finally:
        fm.set_deterministic(False)
    torch.cuda.synchronize()
    assert same_up_to_rounding(o1, o2)
