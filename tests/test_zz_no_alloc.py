"""bsattn_fwd_static: the forward entry point that allocates nothing (its scratch memory is a device
array inside the library) against bsattn_fwd with a caller-provided workspace, through the C ABI.
Two calls in a row share the library's array; the second is smaller, so stale contents of the
first are in the array when it runs."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from helpers import make_qkv, uniform_block_mask, errors, f32, same_up_to_rounding

pytestmark = pytest.mark.gpu


def _both(dev, B, H, N, D, dtype, keep, seed):
    import fa2_custom_mask as fm
    from fa2_custom_mask import _ext
    lib = _ext.lib()
    q, k, v = [x.to(dev) for x in make_qkv(B, H, N, D, dtype, seed)]
    mask = uniform_block_mask(1, 1, N // 64, keep, seed + 1)
    lists = fm.block_mask_to_lists(mask.to(dev))
    sc = 1.0 / np.sqrt(D)
    st = _ext.current_stream(dev)
    outs = []
    for static in (False, True):
        o = torch.full((B, H, N, D), float("nan"), dtype=dtype, device=dev)
        lse = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=dev)
        args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), lists.row_ptr.data_ptr(),
                lists.col_idx.data_ptr(), lists.Bm, lists.Hm, B, H, N, D, _ext.dtype_code(dtype),
                _ext.dtype_code(dtype), float(sc), _ext.strides4(q), _ext.strides4(k), _ext.strides4(v),
                _ext.strides4(o))
        if static:
            # one call first (the library looks up its array's address and sets kernel attributes once per
            # device); then the free memory of the device itself, which any hipMalloc would lower, not only
            # torch's own bookkeeping, must be the same before and after a call
            assert lib.bsattn_fwd_static(*args, st) == 0
            torch.cuda.synchronize()
            free_before, before = torch.cuda.mem_get_info(dev)[0], torch.cuda.memory_allocated(dev)
            rc = lib.bsattn_fwd_static(*args, st)
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info(dev)[0] == free_before and torch.cuda.memory_allocated(dev) == before
        else:
            wsb = _ext.fwd_workspace(B, H, N, D)
            ws = torch.empty(wsb, dtype=torch.uint8, device=dev)
            rc = lib.bsattn_fwd(*args, ws.data_ptr(), wsb, st)
        assert rc == 0, lib.bsattn_strerror(rc)
        torch.cuda.synchronize()
        outs.append((o, lse))
    (o_ws, lse_ws), (o_st, lse_st) = outs
    # against the existing entry point: equal up to the run-to-run rounding of the forward
    # (two rounding steps of the output type: bf16 keeps 8 bits)
    assert same_up_to_rounding(o_st, o_ws, rel=2.0 ** -9 if dtype == torch.float16 else 2.0 ** -6, abs_=3e-4 if dtype == torch.float16 else 2e-3)
    assert np.allclose(lse_st.cpu().numpy(), lse_ws.cpu().numpy(), atol=2e-3)
    # and against the oracle, at the forward's tolerances
    o_ref, lse_ref = orc.naive_attention(f32(q.cpu()), f32(k.cpu()), f32(v.cpu()), mask.numpy(), sc, return_lse=True)
    ma, rl = errors(o_st, o_ref)
    assert ma <= (2e-2 if dtype == torch.float16 else 3e-2) and rl <= (1e-3 if dtype == torch.float16 else 3e-3)
    assert np.abs(lse_st.cpu().numpy() - lse_ref).max() <= 2e-3


def test_static_forward_matches_workspace_forward(dev):
    # first call: one long head, whose row blocks are shared between workgroups (parts and flags in the
    # scratch array are used); second call, smaller, right after it on the same array
    _both(dev, 1, 1, 2048, 64, torch.float16, 0.7, 11)
    _both(dev, 1, 2, 512, 64, torch.float16, 0.5, 12)
    _both(dev, 1, 1, 1024, 128, torch.bfloat16, 0.6, 13)
    # D = 256 with few row blocks: the row lists are shared between workgroups and the scratch array holds
    # their fp32 parts, which a second kernel sums (2 MB here)
    _both(dev, 1, 1, 1024, 256, torch.float16, 0.6, 14)


def test_static_forward_rejects_shapes_beyond_its_scratch(dev):
    from fa2_custom_mask import _ext
    lib = _ext.lib()
    n = ctypes.c_size_t()
    B, H, N, D = 1, 1, 17536, 256        # row lists shared between workgroups: fp32 parts of over 100 MB
    assert lib.bsattn_fwd_workspace(B, H, N, D, ctypes.byref(n)) == 0
    if n.value <= (32 << 20):
        pytest.skip("this shape fits the static scratch on this device")
    P = ctypes.c_void_p(4096)             # never dereferenced: the size check comes first
    s = (ctypes.c_int64 * 4)(H * N * D, N * D, D, 1)
    rc = lib.bsattn_fwd_static(P, P, P, P, None, P, P, 1, 1, B, H, N, D, 0, 0, 0.1, s, s, s, s, None)
    assert rc == -9 and b"static" in lib.bsattn_strerror(rc)
