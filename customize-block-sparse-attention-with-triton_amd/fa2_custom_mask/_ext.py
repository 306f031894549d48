"""ctypes binding of libbsattn.so, the C-ABI library holding the gfx950 kernels.

There is deliberately no fallback: if the library is missing, or a call returns an error
code, a RuntimeError is raised.
"""
import ctypes
import functools
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("BSATTN_LIB", os.path.join(_HERE, "libbsattn.so"))
_lib = None

F16, BF16, F32 = 0, 1, 2
_DTYPE_CODE = {torch.float16: F16, torch.bfloat16: BF16, torch.float32: F32}

_i, _i64, _p, _f = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_float
_SIGNATURES = {
    "bsattn_version": ([], _i),
    "bsattn_set_deterministic": ([_i], _i),
    "bsattn_strerror": ([_i], ctypes.c_char_p),
    "bsattn_reduce_dense_mask": ([_p, _i, _i, _i, _i64, _i64, _i64, _p, _p], _i),
    "bsattn_mask_lists_workspace": ([_i, _i, _i, ctypes.POINTER(ctypes.c_size_t)], _i),
    "bsattn_block_mask_to_lists": ([_p, _i, _i, _i, _i64, _i64, _i64, _i64, _p, _p, _p, _p, _p,
                                    ctypes.c_size_t, _p], _i),
    "bsattn_pack_mask_tiles": ([_p, _i, _i, _i, _i64, _i64, _i64, _i64, _p, _p, _p, _p, _p], _i),
    "bsattn_reduce_pack_dense_mask": ([_p, _i, _i, _i, _i64, _i64, _i64, _p, _p, _p, _p], _i),
    "bsattn_gather_mask_tiles": ([_p, _p, _i, _i, _i, _i, _p, _p, _p, _p, _p], _i),
    "bsattn_tail_mask_tiles": ([_i, _i, _i, _i, _i, _p, _p, _p, _p, _p], _i),
    "bsattn_fwd_workspace": ([_i, _i, _i, _i, ctypes.POINTER(ctypes.c_size_t)], _i),
    "bsattn_fwd": ([_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _f,
                    _p, _p, _p, _p, _p, ctypes.c_size_t, _p], _i),
    "bsattn_fwd_block_mask_workspace": ([_i, _i, _i, _i, _i, _i, ctypes.POINTER(ctypes.c_size_t)], _i),
    "bsattn_fwd_block_mask": ([_p, _p, _p, _p, _p, _p, _p, _i, _i, _p, _p, _p, _i, _i, _i, _i, _i, _i, _f,
                               _p, _p, _p, _p, _p, ctypes.c_size_t, _p], _i),
    "bsattn_fwd_static": ([_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _f,
                           _p, _p, _p, _p, _p], _i),
    "bsattn_fwd_elementwise": ([_p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _f,
                                _p, _p, _p, _p, _p, ctypes.c_size_t, _p], _i),
    "bsattn_bwd_workspace": ([_i, _i, _i, _i, ctypes.POINTER(ctypes.c_size_t)], _i),
    "bsattn_bwd": ([_p] * 13 + [_i] * 8 + [_f] + [_p] * 8 + [_p, ctypes.c_size_t, _p], _i),
    "bsattn_bwd_elementwise": ([_p] * 15 + [_i] * 8 + [_f] + [_p] * 8 + [_p, ctypes.c_size_t, _p], _i),
    "bsattn_reorder": ([_p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _p, _p], _i),
}
EXPORTS = tuple(_SIGNATURES)
ABI_MAJOR = 2      # BSATTN_ABI_VERSION / 100 of the header these signatures were written against


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libbsattn.so not found at %s: build it with "
                "`python customize-block-sparse-attention-with-triton_amd/build.py`" % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(l, name)
            fn.argtypes = argtypes
            fn.restype = restype
        if l.bsattn_version() // 100 != ABI_MAJOR:
            raise RuntimeError("%s has ABI version %d, this package needs %d.x: rebuild it with build.py"
                               % (LIB_PATH, l.bsattn_version(), ABI_MAJOR))
        _lib = l
    return _lib


def check(rc, what):
    if rc != 0:
        raise RuntimeError("%s failed: %s (code %d)" % (what, lib().bsattn_strerror(rc).decode(), rc))


def dtype_code(dt):
    try:
        return _DTYPE_CODE[dt]
    except KeyError:
        raise TypeError("unsupported dtype %s" % dt)


@functools.lru_cache(maxsize=256)
def _strides_array(strides):
    return (ctypes.c_int64 * 4)(*strides)


def strides4(t):
    """Element strides of a 4-d tensor as a C array (cached per stride tuple; never written to)."""
    return _strides_array(t.stride())


def raw_stream(device):
    """The current stream of `device` as its raw handle (an int; 0 is the default stream)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(index)


def current_stream(device):
    return ctypes.c_void_p(raw_stream(device))


@functools.lru_cache(maxsize=256)
def mask_lists_workspace(Bm, Hm, nb):
    n = ctypes.c_size_t()
    check(lib().bsattn_mask_lists_workspace(Bm, Hm, nb, ctypes.byref(n)), "bsattn_mask_lists_workspace")
    return n.value


def _device_index(device):
    """Index of `device` (a torch device or None = the current one); -1 without a GPU."""
    if device is not None and getattr(device, "index", None) is not None:
        return device.index
    return torch.cuda.current_device() if torch.cuda.is_available() else -1


@functools.lru_cache(maxsize=256)
def _workspace_on(which, B, H, N, D, index):
    # the sizes depend on the device the library sees as current (its number of compute units)
    n = ctypes.c_size_t()
    fn = getattr(lib(), which)
    if index >= 0 and index != torch.cuda.current_device():
        with torch.cuda.device(index):
            rc = fn(B, H, N, D, ctypes.byref(n))
    else:
        rc = fn(B, H, N, D, ctypes.byref(n))
    check(rc, which)
    return n.value


@functools.lru_cache(maxsize=256)
def _fused_workspace_on(Bm, Hm, B, H, N, D, index):
    n = ctypes.c_size_t()
    if index >= 0 and index != torch.cuda.current_device():
        with torch.cuda.device(index):
            rc = lib().bsattn_fwd_block_mask_workspace(Bm, Hm, B, H, N, D, ctypes.byref(n))
    else:
        rc = lib().bsattn_fwd_block_mask_workspace(Bm, Hm, B, H, N, D, ctypes.byref(n))
    check(rc, "bsattn_fwd_block_mask_workspace")
    return n.value


def fwd_block_mask_workspace(Bm, Hm, B, H, N, D, device=None):
    return _fused_workspace_on(Bm, Hm, B, H, N, D, _device_index(device))


def fwd_workspace(B, H, N, D, device=None):
    return _workspace_on("bsattn_fwd_workspace", B, H, N, D, _device_index(device))


def bwd_workspace(B, H, N, D, device=None):
    return _workspace_on("bsattn_bwd_workspace", B, H, N, D, _device_index(device))
