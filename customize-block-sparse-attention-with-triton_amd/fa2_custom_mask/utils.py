"""Mask preprocessing on the GPU and small helpers.

`is_hip` / `keep` keep the names exported by the reference (fa2_custom_mask/utils.py:3-14).
"""
import ctypes
import weakref

import torch

from . import _ext

TILE = 64


def is_hip():
    """The reference hard-wires False (fa2_custom_mask/utils.py:3-4); this build only runs on HIP."""
    return True


def keep(conf):
    """Autotune filter of the reference (fa2_custom_mask/utils.py:9-14).  There is no autotuner
    here; every configuration is kept."""
    return True


class TileLists:
    """Device-resident kept-tile lists of a block mask [Bm, Hm, nb, nb] (fixed shapes, no
    host synchronisation): row_ptr int32 [Bm*Hm*nb+1], col_idx int32 [Bm*Hm*nb*nb] (first T
    entries valid), counts int32 [2] = (G, T), groups int32 [Bm*Hm*nb, 5] (first G rows
    valid) or None.  All of them live in one int32 buffer (workspace | row_ptr | counts | col_idx | groups);
    the tensor views are made when first asked for, the calls into the library only need the addresses."""

    __slots__ = ("buf", "Bm", "Hm", "nb", "has_groups", "partial", "bits", "_views",
                 "ws_ptr", "ws_bytes", "row_ptr_ptr", "counts_ptr", "col_idx_ptr", "groups_ptr", "_off")

    def __init__(self, Bm, Hm, nb, device, want_groups=False):
        rows = Bm * Hm * nb
        wsb = _ext.mask_lists_workspace(Bm, Hm, nb)
        o_ptr = (wsb + 3) // 4
        o_counts = o_ptr + rows + 1
        o_cols = o_counts + 2
        o_groups = o_cols + rows * nb
        self.buf = torch.empty(o_groups + (rows * 5 if want_groups else 0), dtype=torch.int32, device=device)
        self.Bm, self.Hm, self.nb, self.has_groups = Bm, Hm, nb, want_groups
        self._off = (o_ptr, o_counts, o_cols, o_groups)
        base = self.buf.data_ptr()
        self.ws_ptr, self.ws_bytes = base, wsb
        self.row_ptr_ptr, self.counts_ptr = base + 4 * o_ptr, base + 4 * o_counts
        self.col_idx_ptr = base + 4 * o_cols
        self.groups_ptr = base + 4 * o_groups if want_groups else None
        # elementwise masks only: per kept tile "partly set" flag and packed 64 x 64 bits
        self.partial, self.bits = None, None
        self._views = None

    def _make_views(self):
        if self._views is None:
            o_ptr, o_counts, o_cols, o_groups = self._off
            b = self.buf
            rows = self.Bm * self.Hm * self.nb
            self._views = (b[o_ptr:o_counts], b[o_counts:o_cols], b[o_cols:o_groups],
                           b[o_groups:].view(rows, 5) if self.has_groups else None)
        return self._views

    @property
    def row_ptr(self):
        return self._make_views()[0]

    @property
    def counts(self):
        return self._make_views()[1]

    @property
    def col_idx(self):
        return self._make_views()[2]

    @property
    def groups(self):
        return self._make_views()[3]


def _check_mask(mask):
    if not isinstance(mask, torch.Tensor) or mask.dtype != torch.bool:
        raise TypeError("mask must be a torch.bool tensor")       # fa2_custom_mask.py:20
    if mask.dim() != 4:
        raise ValueError("mask must have 4 dimensions [B, H, rows, cols]")
    if not mask.is_cuda:
        raise RuntimeError("mask must live on the GPU")


def reduce_dense_mask(mask):
    """Elementwise mask [Bm,Hm,N,N] -> block mask [Bm,Hm,N/64,N/64] (tile kept iff any element
    set; exact inverse of the expansion at kernel-test.py:18 for tile-constant masks)."""
    _check_mask(mask)
    Bm, Hm, N, N2 = mask.shape
    if N != N2 or N % TILE != 0:
        raise ValueError("dense mask must be [.., N, N] with N a multiple of 64")
    if mask.stride(3) != 1 or any(s % 16 for s in mask.stride()[:3]) or mask.data_ptr() % 16:
        mask = mask.contiguous()
    nb = N // TILE
    block = torch.empty((Bm, Hm, nb, nb), dtype=torch.bool, device=mask.device)
    rc = _ext.lib().bsattn_reduce_dense_mask(mask.data_ptr(), Bm, Hm, N, mask.stride(0), mask.stride(1),
                                             mask.stride(2), block.data_ptr(),
                                             _ext.current_stream(mask.device))
    _ext.check(rc, "bsattn_reduce_dense_mask")
    return block


def block_mask_to_lists(block, transpose=False, want_groups=False):
    """Block mask -> TileLists.  transpose=True lists, for every column block, the kept row
    blocks (what the dK/dV pass walks)."""
    _check_mask(block)
    Bm, Hm, nb, nb2 = block.shape
    if nb != nb2:
        raise ValueError("block mask must be square")
    lists = TileLists(Bm, Hm, nb, block.device, want_groups)
    sb, sh, sm, sn = block.stride()
    if transpose:
        sm, sn = sn, sm
    rc = _ext.lib().bsattn_block_mask_to_lists(
        block.data_ptr(), Bm, Hm, nb, sb, sh, sm, sn, lists.row_ptr_ptr, lists.col_idx_ptr,
        lists.groups_ptr, lists.counts_ptr, lists.ws_ptr, lists.ws_bytes, _ext.current_stream(block.device))
    _ext.check(rc, "bsattn_block_mask_to_lists")
    return lists


def pack_mask_tiles(mask, lists, transpose=False):
    """Elementwise mask [Bm,Hm,N,N] + the TileLists of its reduced form -> (tile_partial uint8
    [cap], tile_bits int64 [cap, 64]) with one slot per kept tile: is the tile only partly set,
    and its 64 x 64 bools as 64 words (word r, bit c = element (r, c) of the tile; with
    transpose=True, matching transposed lists, element (c, r))."""
    _check_mask(mask)
    Bm, Hm, N, N2 = mask.shape
    if N != N2 or N % TILE != 0 or N // TILE != lists.nb or (Bm, Hm) != (lists.Bm, lists.Hm):
        raise ValueError("mask and lists do not belong together")
    sb, sh, sm, sn = mask.stride()
    if min(sm, sn) != 1 or any(s % 4 for s in (sb, sh, max(sm, sn))) or mask.data_ptr() % 4:
        mask = mask.contiguous()
        sb, sh, sm, sn = mask.stride()
    if transpose:
        sm, sn = sn, sm
    cap = Bm * Hm * lists.nb * lists.nb
    partial = torch.empty(cap, dtype=torch.uint8, device=mask.device)
    bits = torch.empty((cap, 64), dtype=torch.int64, device=mask.device)
    rc = _ext.lib().bsattn_pack_mask_tiles(mask.data_ptr(), Bm, Hm, N, sb, sh, sm, sn, lists.row_ptr_ptr,
                                           lists.col_idx_ptr, partial.data_ptr(), bits.data_ptr(),
                                           _ext.current_stream(mask.device))
    _ext.check(rc, "bsattn_pack_mask_tiles")
    return partial, bits


def reduce_pack_dense_mask(mask):
    """Elementwise mask [Bm,Hm,N,N] -> (block mask [Bm,Hm,nb,nb], grid_partial uint8 [Bm*Hm*nb*nb], grid_bits int64
    [Bm*Hm*nb*nb, 64]) in one pass over the mask: the reduced mask, and the "partly set" flag and packed words of
    every tile that has a set element, at the tile's position in the grid (gather_mask_tiles brings them into
    list order)."""
    _check_mask(mask)
    Bm, Hm, N, N2 = mask.shape
    if N != N2 or N % TILE != 0:
        raise ValueError("dense mask must be [.., N, N] with N a multiple of 64")
    if mask.stride(3) != 1 or any(s % 16 for s in mask.stride()[:3]) or mask.data_ptr() % 16:
        mask = mask.contiguous()
    nb = N // TILE
    tiles = Bm * Hm * nb * nb
    block = torch.empty((Bm, Hm, nb, nb), dtype=torch.bool, device=mask.device)
    grid_partial = torch.empty(tiles, dtype=torch.uint8, device=mask.device)
    grid_bits = torch.empty((tiles, 64), dtype=torch.int64, device=mask.device)
    rc = _ext.lib().bsattn_reduce_pack_dense_mask(mask.data_ptr(), Bm, Hm, N, mask.stride(0), mask.stride(1),
                                                  mask.stride(2), block.data_ptr(), grid_partial.data_ptr(),
                                                  grid_bits.data_ptr(), _ext.current_stream(mask.device))
    _ext.check(rc, "bsattn_reduce_pack_dense_mask")
    return block, grid_partial, grid_bits


def gather_mask_tiles(grid_partial, grid_bits, lists, transpose=False):
    """(tile_partial, tile_bits) in the format of pack_mask_tiles for `lists` (the row lists, or with
    transpose=True the column lists: words per key, bits per query) from the grid-ordered result of
    reduce_pack_dense_mask."""
    dev = lists.row_ptr.device
    cap = lists.Bm * lists.Hm * lists.nb * lists.nb
    partial = torch.empty(cap, dtype=torch.uint8, device=dev)
    bits = torch.empty((cap, 64), dtype=torch.int64, device=dev)
    rc = _ext.lib().bsattn_gather_mask_tiles(grid_partial.data_ptr(), grid_bits.data_ptr(), lists.Bm, lists.Hm, lists.nb,
                                             1 if transpose else 0, lists.row_ptr_ptr, lists.col_idx_ptr,
                                             partial.data_ptr(), bits.data_ptr(), _ext.current_stream(dev))
    _ext.check(rc, "bsattn_gather_mask_tiles")
    return partial, bits


def tail_mask_tiles(lists, valid_last, transpose=False):
    """Words of the kept tiles of a block mask whose last column block holds only `valid_last`
    real keys (sequence length not a multiple of 64): (tile_partial, tile_bits) in the format of
    pack_mask_tiles, every tile completely set except for the padding keys."""
    dev = lists.row_ptr.device
    cap = lists.Bm * lists.Hm * lists.nb * lists.nb
    partial = torch.empty(cap, dtype=torch.uint8, device=dev)
    bits = torch.empty((cap, 64), dtype=torch.int64, device=dev)
    rc = _ext.lib().bsattn_tail_mask_tiles(lists.Bm, lists.Hm, lists.nb, valid_last, 1 if transpose else 0,
                                           lists.row_ptr_ptr, lists.col_idx_ptr, partial.data_ptr(),
                                           bits.data_ptr(), _ext.current_stream(dev))
    _ext.check(rc, "bsattn_tail_mask_tiles")
    return partial, bits


def num_tiles(N):
    """Row (and column) blocks of a sequence of N tokens; the last one may be partly filled."""
    return -(-N // TILE)


def is_block_form(mask, N):
    """True for the reference's block form [.,.,nb,nb], False for an elementwise [.,.,N,N] mask."""
    nb = num_tiles(N)
    if mask.shape[2] == nb and mask.shape[3] == nb and N != nb:
        return True
    if mask.shape[2] == N and mask.shape[3] == N:
        return False
    raise ValueError("mask shape %s matches neither [.., %d, %d] nor [.., %d, %d]"
                     % (tuple(mask.shape), nb, nb, N, N))


def to_block_mask(mask, N):
    """Accepts the reference's block form [.,.,N/64,N/64] or an elementwise [.,.,N,N] mask
    (N a multiple of 64)."""
    _check_mask(mask)
    return mask if is_block_form(mask, N) else reduce_dense_mask(mask)


class _ListsCache:
    """Kept-tile lists of the most recently used masks.  A static mask (the usual case: one mask
    for every layer and step) is indexed once instead of once per call.  An entry is only used
    for the very tensor object it was built from, and only while that tensor has not been
    written to (autograd's version counter)."""

    def __init__(self, capacity=8):
        self.capacity = capacity
        # (weakref to mask, version, N, transpose, lists, stream the lists were built on), most recent last
        self._entries = []

    @staticmethod
    def _version(mask):
        """The tensor's write counter, or None for a tensor that keeps none (one created under
        torch.inference_mode()): writes to such a tensor cannot be seen, so it is never cached."""
        try:
            return mask._version
        except RuntimeError:
            return None

    def get(self, mask, N, transpose):
        version = self._version(mask)
        if version is None:
            return None
        for i, (ref, ver, n, tr, lists, stream) in enumerate(self._entries):
            if ref() is mask and ver == version and n == N and tr == transpose:
                if i != len(self._entries) - 1:
                    self._entries.append(self._entries.pop(i))
                # the lists were filled by kernels on `stream` (a raw handle): work on another stream waits for
                # what that stream has been given so far (no event is recorded when the lists are made: a mask
                # that changes with every call would pay for it every time)
                if _ext.raw_stream(mask.device) != stream:
                    torch.cuda.current_stream(mask.device).wait_stream(
                        torch.cuda.ExternalStream(stream, device=mask.device) if stream else torch.cuda.default_stream(mask.device))
                return lists
        return None

    def put(self, mask, N, transpose, lists):
        version = self._version(mask)
        if version is None:
            return
        if len(self._entries) >= self.capacity:
            self._entries = [e for e in self._entries if e[0]() is not None][-(self.capacity - 1):]
        self._entries.append((weakref.ref(mask), version, N, transpose, lists, _ext.raw_stream(mask.device)))

    def clear(self):
        self._entries = []
        if "grid_cache" in globals():
            grid_cache.clear()


lists_cache = _ListsCache()


class _GridCache:
    """The grid-ordered words of the most recently used elementwise masks (reduce_pack_dense_mask), so that the
    second form of the lists (the column lists a backward asks for after the forward asked for the row lists)
    does not read the mask again.  Same identity rule as the lists cache; two entries, since one holds as
    many bytes as an eighth of its mask."""

    def __init__(self, capacity=2):
        self.capacity = capacity
        self._entries = []     # (weakref to mask, version, N, (block, grid_partial, grid_bits), stream, event)

    def get(self, mask, N):
        version = _ListsCache._version(mask)
        if version is None:
            return None
        for ref, ver, n, grid, stream, ready in self._entries:
            if ref() is mask and ver == version and n == N:
                current = torch.cuda.current_stream(mask.device)
                if current != stream:
                    current.wait_event(ready)
                return grid
        return None

    def put(self, mask, N, grid):
        version = _ListsCache._version(mask)
        if version is None:
            return
        stream = torch.cuda.current_stream(mask.device)
        ready = torch.cuda.Event()
        ready.record(stream)
        self._entries = [e for e in self._entries if e[0]() is not None]
        self._entries.append((weakref.ref(mask), version, N, grid, stream, ready))
        del self._entries[:-self.capacity]

    def clear(self):
        self._entries = []


grid_cache = _GridCache()


def mask_to_lists(mask, N, transpose=False, both=False):
    """TileLists of a block or elementwise mask for sequence length N, through the cache.  both: the caller will
    also ask for the other orientation (a backward follows): an elementwise mask is then read once for both
    (one pass that packs every tile of the grid, 63 us at N = 17536, against 49 us for the reduction plus 34-78 us
    per orientation for packing the kept tiles from the mask: the one pass wins when both forms are needed or
    most tiles are kept, the two passes when a sparse mask is only used forward)."""
    lists = lists_cache.get(mask, N, transpose)
    if lists is None:
        _check_mask(mask)
        pad = num_tiles(N) * TILE - N          # > 0: q, k, v get `pad` zero rows, whose keys are masked here
        if is_block_form(mask, N):
            lists = block_mask_to_lists(mask, transpose=transpose)
            if pad:
                lists.partial, lists.bits = tail_mask_tiles(lists, TILE - pad, transpose=transpose)
        else:                                  # elementwise form: exact inside tiles
            grid = grid_cache.get(mask, N)
            if grid is None and not (both or transpose):
                dense = torch.nn.functional.pad(mask, (0, pad, 0, pad)) if pad else mask
                lists = block_mask_to_lists(reduce_dense_mask(dense), transpose=transpose)
                lists.partial, lists.bits = pack_mask_tiles(dense, lists, transpose=transpose)
            else:
                if grid is None:
                    dense = torch.nn.functional.pad(mask, (0, pad, 0, pad)) if pad else mask
                    grid = reduce_pack_dense_mask(dense)
                    grid_cache.put(mask, N, grid)
                block, grid_partial, grid_bits = grid
                lists = block_mask_to_lists(block, transpose=transpose)
                lists.partial, lists.bits = gather_mask_tiles(grid_partial, grid_bits, lists, transpose=transpose)
        lists_cache.put(mask, N, transpose, lists)
    return lists
