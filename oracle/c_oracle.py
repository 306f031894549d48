"""ctypes binding of liboracle.so (the C restatement in bsattn_oracle.c).
TEST INFRASTRUCTURE ONLY, like the rest of this directory."""
import ctypes
import os
import subprocess
import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build():
    subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
        _LIB.oracle_num_threads.restype = ctypes.c_int
    return _LIB


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def build_groups(mask):
    mask = np.ascontiguousarray(np.asarray(mask, dtype=np.bool_))
    B, H, nb, _ = mask.shape
    groups = np.empty((B * H * nb, 5), dtype=np.int32)
    n_list = np.empty(max(1, B * H * nb * nb), dtype=np.int32)
    G = ctypes.c_int64(); T = ctypes.c_int64()
    rc = lib().oracle_build_groups(_p(mask.view(np.uint8)), B, H, nb, _p(groups), _p(n_list),
                                   ctypes.byref(G), ctypes.byref(T))
    assert rc == 0
    if G.value == 0:
        return None, None
    return groups[:G.value].copy(), n_list[:T.value].copy()


def num_threads():
    return int(lib().oracle_num_threads())


def naive_fwd(q, k, v, block_mask, sm_scale, row0=0, row1=None, want_lse=True):
    """q,k,v [B,H,N,D] -> (o, lse) fp32; only query rows [row0,row1) are computed."""
    q = np.ascontiguousarray(q, dtype=np.float32); k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    B, H, N, D = q.shape
    bm = np.asarray(block_mask, dtype=np.bool_)
    if bm.shape[0] * bm.shape[1] != 1:
        bm = np.broadcast_to(bm, (B, H) + bm.shape[2:])
    bm = np.ascontiguousarray(bm)
    BHm = bm.shape[0] * bm.shape[1]
    row1 = N if row1 is None else row1
    o = np.zeros((B, H, N, D), dtype=np.float32)
    lse = np.full((B, H, N), -np.inf, dtype=np.float32)
    rc = lib().oracle_naive_fwd(_p(q), _p(k), _p(v), _p(bm.view(np.uint8)), B * H, BHm, N, D,
                                ctypes.c_float(sm_scale), row0, row1, _p(o),
                                _p(lse) if want_lse else None)
    assert rc == 0
    return o, lse


def reorder(x, orders, F, H, W):
    x = np.ascontiguousarray(x); orders = np.ascontiguousarray(orders, dtype=np.int32)
    BS, NH, T, D = x.shape
    out = np.empty_like(x)
    rc = lib().oracle_reorder(_p(x), _p(out), BS, NH, F, H, W, D, x.dtype.itemsize, _p(orders))
    assert rc == 0
    return out


def inv_reorder(x, orders, inv_orders, F, H, W):
    x = np.ascontiguousarray(x); orders = np.ascontiguousarray(orders, dtype=np.int32)
    inv_orders = np.ascontiguousarray(inv_orders, dtype=np.int32)
    BS, NH, T, D = x.shape
    out = np.empty_like(x)
    rc = lib().oracle_inv_reorder(_p(x), _p(out), BS, NH, F, H, W, D, x.dtype.itemsize,
                                  _p(orders), _p(inv_orders))
    assert rc == 0
    return out
