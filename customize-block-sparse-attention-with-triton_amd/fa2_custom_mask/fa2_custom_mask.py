"""Host boundary of the block-sparse attention operator.

Mirrors fa2_custom_mask/fa2_custom_mask.py of the reference: `build_groups_from_block_mask`
(:15-38) and the autograd function behind `flash_attention_custom_mask` (:40-157), with the
device work done by hand-written gfx950 kernels reached through the C ABI in include/bsattn.h.
"""
import collections
import ctypes

import torch

from . import _ext
from .utils import (TILE, TileLists, block_mask_to_lists, lists_cache, mask_to_lists, num_tiles, is_block_form,
                    _check_mask)


def build_groups_from_block_mask(mask):
    """Same contract as the reference (fa2_custom_mask.py:15-38): bool [B,H,nb,nb] ->
    (groups int32 [G,5] = (b,h,m_block,start,length), n_list int32 [T]) on mask.device, rows
    without a kept tile omitted, (None, None) if nothing is kept.  The lists are produced by
    the GPU kernels; only the two sizes G and T are read back to shape the result."""
    assert mask.dtype == torch.bool                                   # :20
    _check_mask(mask)
    lists = block_mask_to_lists(mask, want_groups=True)
    G, T = lists.counts.tolist()
    if G == 0:                                                        # :34-35
        return None, None
    return lists.groups[:G].contiguous(), lists.col_idx[:T].contiguous()   # :36-38


def _prep(x):
    """Kernels need unit stride along the head dimension and 16-byte aligned rows."""
    if x.is_contiguous() and (x.shape[3] * x.element_size()) % 16 == 0 and x.data_ptr() % 16 == 0:
        return x                                                # (the usual case, decided without looking at strides)
    if x.stride(3) != 1 or any((s * x.element_size()) % 16 for s in x.stride()[:3]) or x.data_ptr() % 16:
        return x.contiguous()
    return x


_workspaces = collections.OrderedDict()
WORKSPACE_CACHE_STREAMS = 8          # (device, stream) pairs whose workspace is kept
WORKSPACE_CACHE_BYTES = 256 << 20    # a larger workspace serves its call and is then given back


def clear_workspaces():
    """Gives back the workspaces kept for reuse."""
    _workspaces.clear()


def _workspace(nbytes, device):
    """Scratch memory for one call, kept per (device, stream) and reused by the next call on that stream:
    the kernels need no particular contents on entry, and calls on one stream run one after the
    other.  The cache is bounded (the least recently used stream's workspace goes first, a workspace above
    WORKSPACE_CACHE_BYTES is not kept), and nothing is kept or taken from it while a graph is being captured:
    memory first allocated under capture belongs to the graph's pool.  (Plans own their workspaces: they may be
    replayed from graphs on any stream.)"""
    raw = _ext.raw_stream(device)
    handle = ctypes.c_void_p(raw)
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device), handle
    key = (device.index, raw)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        if nbytes <= WORKSPACE_CACHE_BYTES:
            _workspaces[key] = ws
            while len(_workspaces) > WORKSPACE_CACHE_STREAMS:
                _workspaces.popitem(last=False)
    if key in _workspaces:
        _workspaces.move_to_end(key)
    return ws, handle


def _like(x, dtype):
    """A result tensor laid out as the reference's torch.empty_like(x) lays it out (fa2_custom_mask.py:59,
    101-103): the dimension order of x by stride, without gaps.  For q, k, v sliced out of one packed
    [B, N, 3, H, D] tensor that is [B, N, H, D] order behind a [B, H, N, D] shape."""
    t = torch.empty_like(x, dtype=dtype)
    if x.is_contiguous() and x.shape[3] % 8 == 0:
        return t
    if t.stride(3) != 1 or any((s * t.element_size()) % 16 for s in t.stride()[:3]):
        t = torch.empty(x.shape, dtype=dtype, device=x.device)
    return t


def _check_qkv(q, k, v, mask):
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise RuntimeError("q, k, v must be GPU tensors (there is no CPU path)")
    if q.dim() != 4 or k.shape != q.shape or v.shape != q.shape:
        raise ValueError("q, k, v must share one shape [B, H, N, D]")   # :53-57
    if q.dtype not in (torch.float16, torch.bfloat16) or k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("q, k, v must all be float16 or all bfloat16")
    B, H, N, D = q.shape
    if D not in (16, 32, 64, 128, 256):                                # :58
        raise ValueError("head dimension must be 16, 32, 64, 128 or 256")
    if N < 1:
        raise ValueError("empty sequence")
    if mask is None:
        return B, H, N, D
    _check_mask(mask)
    if mask.shape[0] not in (1, B) or mask.shape[1] not in (1, H):
        raise ValueError("mask batch/head sizes must be 1 or match q")
    is_block_form(mask, N)                                              # raises on any other shape
    return B, H, N, D


def _padded(x, N, D):
    """The kernels work on whole 64-token tiles and on head dimensions 64 and 128: other shapes
    are embedded in zeros.  Zero columns change neither q k^T nor the real columns of the
    output; the keys of zero rows are masked (utils.mask_to_lists), their query rows are dropped."""
    Np, Dp = num_tiles(N) * TILE, (64 if D < 64 else D)
    if (Np, Dp) == (x.shape[2], x.shape[3]):
        return x
    xp = x.new_zeros((x.shape[0], x.shape[1], Np, Dp))
    xp[:, :, :x.shape[2], :x.shape[3]] = x
    return xp


_all_true = {}


def _dense_mask(device, nb):
    """mask=None means plain dense attention (the reference advertises the default but crashes on
    it: `groups` is unbound at fa2_custom_mask.py:69): one all-true block mask shared by all heads."""
    key = (device, nb)
    if key not in _all_true:
        with torch.inference_mode(False):    # an ordinary tensor also when first asked for in inference mode: its lists are cached
            _all_true[key] = torch.ones((1, 1, nb, nb), dtype=torch.bool, device=device)
    return _all_true[key]


def set_deterministic(on):
    """Process-wide switch (bsattn_set_deterministic), returns the previous setting.  On: two runs of the
    forward on the same inputs give the same bits; off (the default): the tiles of a row block go to
    the wavefronts as they become free, which is faster and changes the last bits from run to run.
    The backward is deterministic either way."""
    return bool(_ext.lib().bsattn_set_deterministic(1 if on else 0))


def _plain(q, k, v):
    """q, k, v of one shape without gaps and 16-byte aligned: one stride array serves all three and a result
    laid out like them (the usual case, decided without looking at strides)."""
    return (q.is_contiguous() and k.is_contiguous() and v.is_contiguous() and q.shape[3] % 8 == 0
            and (q.data_ptr() | k.data_ptr() | v.data_ptr()) % 16 == 0)


def _operands(q, k, v, out_dtype):
    """(q, k, v, o, their four stride arrays) as the library takes them."""
    if _plain(q, k, v):
        o = torch.empty_like(q, dtype=out_dtype)                                # :59
        sq = _ext.strides4(q)
        return q, k, v, o, (sq, sq, sq, sq)
    q, k, v = _prep(q), _prep(k), _prep(v)
    o = _like(q, out_dtype)                                                     # :59
    return q, k, v, o, (_ext.strides4(q), _ext.strides4(k), _ext.strides4(v), _ext.strides4(o))


def _forward(q, k, v, lists, sm_scale, out_dtype, want_lse):
    B, H, N, D = q.shape
    q, k, v, o, strides = _operands(q, k, v, out_dtype)
    lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device) if want_lse else None  # :70
    wsb = _ext.fwd_workspace(B, H, N, D, q.device)
    ws, stream = _workspace(wsb, q.device)
    common = (lists.Bm, lists.Hm, B, H, N, D, _ext.dtype_code(q.dtype), _ext.dtype_code(out_dtype), float(sm_scale),
              *strides, ws.data_ptr(), wsb, stream)
    ptrs = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr() if want_lse else None,
            lists.row_ptr_ptr, lists.col_idx_ptr)
    if lists.bits is None:
        rc = _ext.lib().bsattn_fwd(*ptrs, *common)
    else:                                      # elementwise mask: exact inside partly set tiles
        rc = _ext.lib().bsattn_fwd_elementwise(*ptrs, lists.partial.data_ptr(), lists.bits.data_ptr(), *common)
    _ext.check(rc, "bsattn_fwd")
    return o, lse


class ForwardPlan:
    """A forward call with every buffer allocated and every C argument marshalled once; run()
    only enqueues the kernels.  For loops that repeat the same shapes (serving, benchmarks)."""

    def __init__(self, q, k, v, lists, sm_scale, out_dtype=None, stream=None):
        B, H, N, D = q.shape
        if N % TILE or D not in (64, 128, 256):
            raise ValueError("a plan takes whole tiles only: N % 64 == 0 and D in {64, 128, 256}")
        self.q, self.k, self.v, self.lists = _prep(q), _prep(k), _prep(v), lists
        out_dtype = out_dtype or q.dtype
        self.o = _like(self.q, out_dtype)
        self.lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
        wsb = _ext.fwd_workspace(B, H, N, D, q.device)
        self.ws = torch.empty(wsb, dtype=torch.uint8, device=q.device)
        self._keep = (_ext.strides4(self.q), _ext.strides4(self.k), _ext.strides4(self.v), _ext.strides4(self.o))
        stream = stream if stream is not None else torch.cuda.current_stream(q.device)
        tail = (lists.Bm, lists.Hm, B, H, N, D, _ext.dtype_code(q.dtype), _ext.dtype_code(out_dtype),
                float(sm_scale)) + self._keep + (self.ws.data_ptr(), wsb, ctypes.c_void_p(stream.cuda_stream))
        head = (self.q.data_ptr(), self.k.data_ptr(), self.v.data_ptr(), self.o.data_ptr(), self.lse.data_ptr(),
                lists.row_ptr_ptr)
        if lists.bits is not None:
            raise ValueError("a plan takes block masks only")
        self._args = head + (lists.col_idx_ptr,) + tail
        self._fn = _ext.lib().bsattn_fwd

    def run(self):
        rc = self._fn(*self._args)
        if rc != 0:
            _ext.check(rc, "bsattn_fwd")
        return self.o, self.lse


def _backward(q, k, v, o, do, lse, lists, lists_t, sm_scale, out_dtype):
    B, H, N, D = q.shape
    q, k, v, o, do = _prep(q), _prep(k), _prep(v), _prep(o), _prep(do)
    dq, dk, dv = _like(q, out_dtype), _like(k, out_dtype), _like(v, out_dtype)   # :101-103
    wsb = _ext.bwd_workspace(B, H, N, D, q.device)
    ws, stream = _workspace(wsb, q.device)
    tensors = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), do.data_ptr(), lse.data_ptr(),
               dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
               lists.row_ptr_ptr, lists.col_idx_ptr, lists_t.row_ptr_ptr,
               lists_t.col_idx_ptr)
    common = (lists.Bm, lists.Hm, B, H, N, D,
              _ext.dtype_code(q.dtype), _ext.dtype_code(out_dtype), float(sm_scale),
              _ext.strides4(q), _ext.strides4(k), _ext.strides4(v), _ext.strides4(o), _ext.strides4(do),
              _ext.strides4(dq), _ext.strides4(dk), _ext.strides4(dv),
              ws.data_ptr(), wsb, stream)
    if lists.bits is None:
        rc = _ext.lib().bsattn_bwd(*tensors, *common)
    else:                                      # elementwise mask
        rc = _ext.lib().bsattn_bwd_elementwise(*tensors, lists.bits.data_ptr(), lists_t.bits.data_ptr(), *common)
    _ext.check(rc, "bsattn_bwd")
    return dq, dk, dv


class BackwardPlan:
    """The backward counterpart of ForwardPlan: dq, dk, dv and the workspace allocated once, the C
    arguments marshalled once; run() only enqueues the kernels.  o and lse are the forward's
    results for the same q, k, v; block masks only."""

    def __init__(self, q, k, v, o, do, lse, lists, lists_t, sm_scale, out_dtype=None, stream=None):
        B, H, N, D = q.shape
        if N % TILE or D not in (64, 128, 256) or lists.bits is not None:
            raise ValueError("a plan takes whole tiles and block masks only: N % 64 == 0 and D in {64, 128, 256}")
        self.q, self.k, self.v, self.o, self.do = _prep(q), _prep(k), _prep(v), _prep(o), _prep(do)
        self.lse, self.lists, self.lists_t = lse, lists, lists_t
        out_dtype = out_dtype or q.dtype
        self.dq, self.dk, self.dv = _like(self.q, out_dtype), _like(self.k, out_dtype), _like(self.v, out_dtype)
        wsb = _ext.bwd_workspace(B, H, N, D, q.device)
        self.ws = torch.empty(wsb, dtype=torch.uint8, device=q.device)
        self._keep = tuple(_ext.strides4(t) for t in (self.q, self.k, self.v, self.o, self.do, self.dq, self.dk, self.dv))
        stream = stream if stream is not None else torch.cuda.current_stream(q.device)
        self._args = (self.q.data_ptr(), self.k.data_ptr(), self.v.data_ptr(), self.o.data_ptr(), self.do.data_ptr(),
                      lse.data_ptr(), self.dq.data_ptr(), self.dk.data_ptr(), self.dv.data_ptr(),
                      lists.row_ptr_ptr, lists.col_idx_ptr, lists_t.row_ptr_ptr,
                      lists_t.col_idx_ptr, lists.Bm, lists.Hm, B, H, N, D, _ext.dtype_code(q.dtype),
                      _ext.dtype_code(out_dtype), float(sm_scale)) + self._keep + (
                          self.ws.data_ptr(), wsb, ctypes.c_void_p(stream.cuda_stream))
        self._fn = _ext.lib().bsattn_bwd

    def run(self):
        rc = self._fn(*self._args)
        if rc != 0:
            _ext.check(rc, "bsattn_bwd")
        return self.dq, self.dk, self.dv


def _forward_from_block_mask(q, k, v, mask, sm_scale, out_dtype, want_lse):
    """Lists and forward from one call into the library (bsattn_fwd_block_mask), for a block mask whose lists
    are not in the cache: one buffer for the lists, one for the result, and the stream's workspace."""
    B, H, N, D = q.shape
    Bm, Hm, nb = mask.shape[0], mask.shape[1], mask.shape[2]
    q, k, v, o, strides = _operands(q, k, v, out_dtype)
    lists = TileLists(Bm, Hm, nb, q.device)
    lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device) if want_lse else None
    wsb = _ext.fwd_block_mask_workspace(Bm, Hm, B, H, N, D, q.device)
    ws, stream = _workspace(wsb, q.device)
    rc = _ext.lib().bsattn_fwd_block_mask(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr() if want_lse else None,
        mask.data_ptr(), _ext.strides4(mask), Bm, Hm, lists.row_ptr_ptr, lists.col_idx_ptr, lists.counts_ptr,
        B, H, N, D, _ext.dtype_code(q.dtype), _ext.dtype_code(out_dtype), float(sm_scale),
        *strides, ws.data_ptr(), wsb, stream)
    _ext.check(rc, "bsattn_fwd_block_mask")
    return o, lse, lists


def _forward_only(q, k, v, mask, sm_scale, out_fp32, return_lse):
    """The forward of _attention without anything kept for a backward."""
    B, H, N, D = _check_qkv(q, k, v, mask)
    if mask is None:
        mask = _dense_mask(q.device, num_tiles(N))
    out_dtype = torch.float32 if out_fp32 else q.dtype
    whole = N % TILE == 0 and D >= 64
    lists = lists_cache.get(mask, N, False)
    if lists is None and whole and mask.shape[2] * TILE == N:
        # a block mask seen for the first time (or one that changes with every call): lists and forward in one call
        o, lse, lists = _forward_from_block_mask(q, k, v, mask, sm_scale, out_dtype, return_lse)
        lists_cache.put(mask, N, False, lists)
        return (o, lse) if return_lse else o
    if lists is None:
        lists = mask_to_lists(mask, N)
    if whole:
        o, lse = _forward(q, k, v, lists, sm_scale, out_dtype, return_lse)
        return (o, lse) if return_lse else o
    q, k, v = _padded(q, N, D), _padded(k, N, D), _padded(v, N, D)
    o, lse = _forward(q, k, v, lists, sm_scale, out_dtype, return_lse)
    if o.shape[2:] != (N, D):
        o, lse = o[:, :, :N, :D], (lse[:, :, :N] if lse is not None else None)
    return (o, lse) if return_lse else o


class _attention(torch.autograd.Function):
    """forward(q, k, v, mask, sm_scale) as the reference (fa2_custom_mask.py:43-94); two extra
    trailing arguments select an fp32 output and the LSE as second result."""

    @staticmethod
    def forward(ctx, q, k, v, mask=None, sm_scale=1.3, out_fp32=False, return_lse=False):
        B, H, N, D = _check_qkv(q, k, v, mask)
        if mask is None:
            mask = _dense_mask(q.device, num_tiles(N))
        # (a backward will ask for the column lists too when a gradient is wanted)
        lists = mask_to_lists(mask, N, both=any(ctx.needs_input_grad[:3]))   # :48
        out_dtype = torch.float32 if out_fp32 else q.dtype
        q, k, v = _padded(q, N, D), _padded(k, N, D), _padded(v, N, D)
        o, lse = _forward(q, k, v, lists, sm_scale, out_dtype, True)
        ctx.save_for_backward(q, k, v, o, lse, mask)                         # :89
        ctx.lists = lists
        ctx.sm_scale = sm_scale
        ctx.out_dtype = out_dtype
        ctx.return_lse = return_lse
        ctx.shape = (N, D)
        if o.shape[2:] != (N, D):
            o, lse = o[:, :, :N, :D], lse[:, :, :N]
        if return_lse:
            ctx.mark_non_differentiable(lse)
            return o, lse
        return o                                                              # :94

    @staticmethod
    def backward(ctx, do, *unused):
        q, k, v, o, lse, mask = ctx.saved_tensors
        N, D = ctx.shape
        lists_t = mask_to_lists(mask, N, transpose=True)
        o_in = o if o.dtype == q.dtype else o.to(q.dtype)
        do_in = _padded(do if do.dtype == q.dtype else do.to(q.dtype), N, D)
        # autograd hands gradients back in the dtype of q, k, v
        dq, dk, dv = _backward(q, k, v, o_in, do_in, lse, ctx.lists, lists_t, ctx.sm_scale, q.dtype)
        if dq.shape[2:] != (N, D):
            dq, dk, dv = dq[:, :, :N, :D], dk[:, :, :N, :D], dv[:, :, :N, :D]
        return dq, dk, dv, None, None, None, None                            # :155


def flash_attention_custom_mask(q, k, v, mask=None, sm_scale=1.3):
    """Drop-in for the reference's `flash_attention_custom_mask = _attention.apply`
    (fa2_custom_mask.py:157): q,k,v [B,H,N,D] fp16/bf16 on the GPU, mask bool
    [B|1,H|1,nb,nb] with nb = ceil(N/64) (or elementwise [B|1,H|1,N,N]; None = dense attention),
    returns o like q.  D is 16, 32, 64, 128 or 256; N need not be a multiple of 64 (the last block of a
    block mask then covers the remaining tokens).  Shapes other than D in {64,128,256}, N % 64 == 0
    cost one zero-padded copy of q, k, v per call.  The kept-tile lists of a mask tensor are cached
    until the tensor is modified.  When no gradient can be asked for (gradients disabled, or none of q, k, v
    requires one) the call does not go through torch.autograd.Function, which costs about as much host time
    as everything else in a small call."""
    if not (torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)):
        return _forward_only(q, k, v, mask, sm_scale, False, False)
    return _attention.apply(q, k, v, mask, sm_scale)


def flash_attention_custom_mask_lse(q, k, v, mask, sm_scale, out_fp32=False):
    """Same operator, also returning the natural-log logsumexp [B,H,N] fp32 of the kept scaled
    scores; out_fp32=True returns O in fp32.  (Not in the reference, whose second output M is
    only the running maximum: fa2_fwd.py:194-196.)"""
    if not (torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)):
        return _forward_only(q, k, v, mask, sm_scale, out_fp32, True)
    return _attention.apply(q, k, v, mask, sm_scale, out_fp32, True)


def attention_forward_backward(q, k, v, mask, sm_scale, do, out_fp32=False):
    """Non-autograd entry: (o, lse, dq, dk, dv) in one call; with out_fp32 all five results
    are fp32 (autograd itself can only hand back gradients in the dtype of q)."""
    B, H, N, D = _check_qkv(q, k, v, mask)
    if mask is None:
        mask = _dense_mask(q.device, num_tiles(N))
    lists = mask_to_lists(mask, N, both=True)
    lists_t = mask_to_lists(mask, N, transpose=True)
    out_dtype = torch.float32 if out_fp32 else q.dtype
    q, k, v = _padded(q, N, D), _padded(k, N, D), _padded(v, N, D)
    o, lse = _forward(q, k, v, lists, sm_scale, out_dtype, True)
    o_in = o if o.dtype == q.dtype else o.to(q.dtype)
    dq, dk, dv = _backward(q, k, v, o_in, _padded(do.to(q.dtype), N, D), lse, lists, lists_t, sm_scale, out_dtype)
    if o.shape[2:] != (N, D):
        o, lse = o[:, :, :N, :D], lse[:, :, :N]
        dq, dk, dv = dq[:, :, :N, :D], dk[:, :, :N, :D], dv[:, :, :N, :D]
    return o, lse, dq, dk, dv
