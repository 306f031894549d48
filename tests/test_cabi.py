"""C-ABI checks that need no GPU: the library loads, exports every declared symbol, and
rejects bad arguments before any device work."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from fa2_custom_mask import _ext
    header = open(os.path.join(ROOT, "include", "bsattn.h")).read()
    declared = set(re.findall(r"\b(bsattn_[a-z_0-9]+)\s*\(", header))
    assert declared == set(_ext.EXPORTS)
    lib = ctypes.CDLL(_ext.LIB_PATH)
    for name in declared:
        assert getattr(lib, name) is not None
    assert _ext.lib().bsattn_version() // 100 == _ext.ABI_MAJOR
    assert int(re.search(r"#define BSATTN_ABI_VERSION (\d+)", header).group(1)) == _ext.lib().bsattn_version()


def test_strerror():
    from fa2_custom_mask import _ext
    l = _ext.lib()
    assert l.bsattn_strerror(0) == b"ok"
    msgs = {l.bsattn_strerror(c) for c in range(-9, 1)}
    assert len(msgs) == 10 and b"unknown error code" not in msgs
    assert l.bsattn_strerror(-99) == b"unknown error code"


def test_argument_validation_without_gpu():
    from fa2_custom_mask import _ext
    l = _ext.lib()
    n = ctypes.c_size_t()
    ok = (ctypes.c_int64 * 4)(64 * 64, 64 * 64, 64, 1)
    P = ctypes.c_void_p(4096)                     # never dereferenced: validation fails first
    def fwd(**kw):
        a = dict(q=P, k=P, v=P, o=P, lse=None, rp=P, ci=P, Bm=1, Hm=1, B=1, H=1, N=64, D=64, dt=0, odt=0,
                 qs=ok, ks=ok, vs=ok, os=ok, ws=P, wsb=1 << 40)
        a.update(kw)
        return l.bsattn_fwd(a["q"], a["k"], a["v"], a["o"], a["lse"], a["rp"], a["ci"], a["Bm"], a["Hm"],
                            a["B"], a["H"], a["N"], a["D"], a["dt"], a["odt"], 0.125, a["qs"], a["ks"],
                            a["vs"], a["os"], a["ws"], a["wsb"], None)
    assert fwd(q=None) == -1 and fwd(rp=None) == -1
    assert fwd(N=100) == -2 and fwd(B=0) == -2 and fwd(Bm=3, B=2) == -2
    assert fwd(dt=5) == -3 and fwd(odt=1) == -3
    assert fwd(D=96) == -4 and fwd(D=512) == -4
    bad = (ctypes.c_int64 * 4)(64 * 64, 64 * 64, 64, 2)
    assert fwd(qs=bad) == -5
    odd = (ctypes.c_int64 * 4)(64 * 68, 64 * 68, 68, 1)
    assert fwd(ks=odd) == -5
    assert fwd(q=ctypes.c_void_p(4098)) == -5
    assert fwd(ws=None) == -6 and fwd(wsb=16) == -6
    assert l.bsattn_fwd_workspace(1, 1, 100, 64, ctypes.byref(n)) == -2
    assert l.bsattn_fwd_workspace(1, 1, 128, 64, None) == -1
    assert l.bsattn_fwd_workspace(1, 1, 17536, 64, ctypes.byref(n)) == 0 and n.value > 0
    assert l.bsattn_mask_lists_workspace(1, 1, 274, ctypes.byref(n)) == 0 and n.value == 274 * 8
    assert l.bsattn_mask_lists_workspace(1, 1, 0, ctypes.byref(n)) == -2
    assert l.bsattn_mask_lists_workspace(64, 64, 4096, ctypes.byref(n)) == -8
    assert l.bsattn_reduce_dense_mask(None, 1, 1, 64, 0, 0, 64, P, None) == -1
    assert l.bsattn_reduce_dense_mask(P, 1, 1, 65, 0, 0, 80, P, None) == -2
    assert l.bsattn_reduce_dense_mask(P, 1, 1, 64, 0, 0, 72, P, None) == -5
    assert l.bsattn_block_mask_to_lists(P, 1, 1, 4, 16, 16, 4, 1, P, P, None, P, None, 0, None) == -6
    assert l.bsattn_block_mask_to_lists(P, 1, 1, 4, 16, 16, 4, 1, None, P, None, P, P, 64, None) == -1
    assert l.bsattn_tail_mask_tiles(1, 1, 4, 0, 0, P, P, P, P, None) == -2       # 1..64 valid keys
    assert l.bsattn_tail_mask_tiles(1, 1, 4, 65, 0, P, P, P, P, None) == -2
    assert l.bsattn_tail_mask_tiles(1, 1, 4, 10, 0, P, None, P, P, None) == -1
    assert l.bsattn_reorder(P, P, 1, 1, 2, 2, 2, 3, 2, P, None, None) == -5      # 6-byte rows
    assert l.bsattn_reorder(P, P, 1, 1, 0, 2, 2, 4, 2, P, None, None) == -2
    assert l.bsattn_reorder(P, P, 1, 1, 2, 2, 2, 4, 2, None, None, None) == -1


def test_python_wrapper_rejects_bad_input_without_gpu():
    import torch
    import fa2_custom_mask as fm
    q = torch.zeros(1, 1, 128, 64, dtype=torch.float16)
    m = torch.ones(1, 1, 2, 2, dtype=torch.bool)
    with pytest.raises(RuntimeError):
        fm.flash_attention_custom_mask(q, q, q, m, 0.125)                        # CPU tensors: no CPU path
    with pytest.raises(AssertionError):                                          # fa2_custom_mask.py:20
        fm.build_groups_from_block_mask(torch.ones(1, 1, 2, 2))
    with pytest.raises(RuntimeError):
        fm.build_groups_from_block_mask(m)                                       # CPU mask: no CPU path

