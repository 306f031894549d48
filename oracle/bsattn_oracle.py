"""CPU oracle for the block-sparse attention path.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only the test-suite, the smoke
entry and the CPU-baseline leg of the benchmark may import it.  The shipped
operator never calls into it and has no CPU fallback.

It restates, in numpy, what the reference computes on this path.  Every
function cites the reference lines it follows (paths are relative to the
reference repository root).

How each function is pinned (see tests/test_oracle_*.py):
  build_groups_from_block_mask  hand-worked fixture (tests/golden/groups_fixture.json),
                                torch.nonzero + cumsum closed form, structural
                                invariants, special masks (dense / identity / tril).
  naive_attention               torch.nn.functional.scaled_dot_product_attention (dense
                                and boolean-mask forms), v=const / k=0 closed forms,
                                block-diagonal decomposition.
  tiled_attention               equality with naive_attention in float64 (pins the
                                online-softmax recurrence), order invariance.
  logsumexp                     torch.logsumexp of the masked scaled scores.
  attention_backward            torch.autograd through the naive fp32/fp64 path,
                                central finite differences in float64, rowsum(dS)=0.
  reorder / inv_reorder         torch view/permute/reshape closed form, round trip.
No function here is "parity unpinned".
"""
import numpy as np

TILE = 64                      # fixed 64x64 tiles: fa2_custom_mask/fa2_fwd.py:13-14
LOG2E = 1.44269504             # the constant the reference folds in: fa2_custom_mask/fa2_fwd.py:150


# ----------------------------------------------------------------------------
# mask -> kept-tile index lists
# ----------------------------------------------------------------------------
def build_groups_from_block_mask(mask):
    """Follows fa2_custom_mask/fa2_custom_mask.py:15-38 with plain loops.

    mask: bool array [B, H, nb, nb].  Returns (groups int32 [G,5], n_list int32 [T])
    with groups[g] = (b, h, m_block, start, length); rows without a kept tile are
    omitted (:29-30); (None, None) when nothing is kept (:34-35).
    """
    mask = np.asarray(mask)
    assert mask.dtype == np.bool_ and mask.ndim == 4          # :20-21
    B, H, nb, nb2 = mask.shape
    groups, n_list = [], []
    for b in range(B):                                        # :24
        for h in range(H):                                    # :25
            for m in range(nb):                               # :27
                row = mask[b, h, m]
                active = [n for n in range(nb2) if row[n]]    # :28 nonzero, ascending
                if not active:                                # :29-30
                    continue
                start = len(n_list)                           # :31
                n_list.extend(active)                         # :32
                groups.append([b, h, m, start, len(active)])  # :33
    if not groups:                                            # :34-35
        return None, None
    return (np.asarray(groups, dtype=np.int32).reshape(-1, 5),
            np.asarray(n_list, dtype=np.int32))               # :36-38


def csr_from_block_mask(mask):
    """Fixed-shape form of the same lists: row_ptr [B*H*nb+1], col_idx [T].

    Same traversal as build_groups_from_block_mask (fa2_custom_mask.py:24-33) but empty
    rows keep a zero-length entry, so row r = (b*H+h)*nb+m is addressable directly.
    """
    mask = np.asarray(mask, dtype=np.bool_)
    B, H, nb, nb2 = mask.shape
    counts = mask.reshape(B * H * nb, nb2).sum(axis=1)
    row_ptr = np.zeros(B * H * nb + 1, dtype=np.int32)
    row_ptr[1:] = np.cumsum(counts)
    col_idx = np.nonzero(mask.reshape(-1, nb2))[1].astype(np.int32)
    return row_ptr, col_idx


def csc_from_block_mask(mask):
    """Column lists for the backward pass: for every (b,h,n) the ascending kept row blocks."""
    mask = np.asarray(mask, dtype=np.bool_)
    return csr_from_block_mask(np.swapaxes(mask, 2, 3))


def expand_block_mask(block):
    """Block mask -> elementwise mask, kernel-test.py:18 (repeat_interleave(64) twice)."""
    block = np.asarray(block, dtype=np.bool_)
    return np.repeat(np.repeat(block, TILE, axis=-2), TILE, axis=-1)


def reduce_dense_mask(dense):
    """Elementwise mask [.., N, N] -> block mask [.., N/64, N/64]; a tile is kept iff any
    element in it is set (inverse of kernel-test.py:18 for tile-constant masks)."""
    dense = np.asarray(dense, dtype=np.bool_)
    *lead, N, N2 = dense.shape
    assert N % TILE == 0 and N2 % TILE == 0
    t = dense.reshape(*lead, N // TILE, TILE, N2 // TILE, TILE)
    return t.any(axis=(-3, -1))


# ----------------------------------------------------------------------------
# naive masked softmax attention (the parity bar)
# ----------------------------------------------------------------------------
def _bcast_mask(block_mask, B, H):
    block_mask = np.asarray(block_mask, dtype=np.bool_)
    assert block_mask.ndim == 4
    return np.broadcast_to(block_mask, (B, H) + block_mask.shape[2:])


def _keep_rows(mask_bh, N, r0, r1):
    """Elementwise keep matrix of query rows [r0, r1): the mask of one head is either a block
    mask [N/64, N/64] (expanded as kernel-test.py:18) or already elementwise [N, N]."""
    if mask_bh.shape[-1] == N and N != N // TILE:
        return mask_bh[r0:r1]
    return np.repeat(np.repeat(mask_bh[r0 // TILE:r1 // TILE], TILE, 0), TILE, 1)


def pack_mask_tiles(dense, transpose=False):
    """Data format of the elementwise-mask path (no counterpart in the reference): for every
    kept tile of the reduced mask, in list order (row lists, or column lists with
    transpose=True): partial flag (tile not completely set) and 64 words, word r bit c =
    element (r, c) of the tile (element (c, r) with transpose=True).  Plain loops."""
    dense = np.asarray(dense, dtype=bool)
    Bm, Hm, N, _ = dense.shape
    nb = N // TILE
    partial, words = [], []
    for b in range(Bm):
        for h in range(Hm):
            for a in range(nb):
                for c in range(nb):
                    rb, cb = (c, a) if transpose else (a, c)
                    t = dense[b, h, rb * TILE:(rb + 1) * TILE, cb * TILE:(cb + 1) * TILE]
                    if not t.any():
                        continue
                    if transpose:
                        t = t.T
                    partial.append(0 if t.all() else 1)
                    words.append([sum(int(t[r, cc]) << cc for cc in range(TILE)) for r in range(TILE)])
    return np.array(partial, dtype=np.uint8), np.array(words, dtype=np.uint64).reshape(-1, TILE)


def naive_attention(q, k, v, block_mask, sm_scale, dtype=np.float32, row_chunk=2048,
                    return_lse=False):
    """kernel-test.py:37-40: attn = q@k^T*sm_scale; masked_fill(~mask,-inf); softmax; attn@v.

    q,k,v: [B,H,N,D] arrays (any float dtype; upcast to `dtype`).  block_mask:
    [B|1, H|1, N/64, N/64] bool, expanded as kernel-test.py:18, or an elementwise
    [B|1, H|1, N, N] bool mask used as it is.  Query rows are processed
    in chunks, which is exact for a row-wise softmax.  Rows without any kept key give
    O = 0 and lse = -inf here (the reference's naive path gives NaN, its kernel leaves
    the row unwritten: fa2_custom_mask.py:29-30,59).
    """
    q = np.asarray(q, dtype=dtype); k = np.asarray(k, dtype=dtype); v = np.asarray(v, dtype=dtype)
    B, H, N, D = q.shape
    bm = _bcast_mask(block_mask, B, H)
    out = np.zeros((B, H, N, v.shape[-1]), dtype=dtype)
    lse = np.full((B, H, N), -np.inf, dtype=dtype)
    row_chunk = max(TILE, (row_chunk // TILE) * TILE)
    for b in range(B):
        for h in range(H):
            kt = k[b, h].T
            for r0 in range(0, N, row_chunk):
                r1 = min(N, r0 + row_chunk)
                s = (q[b, h, r0:r1] @ kt) * dtype(sm_scale)                    # :37
                keep = _keep_rows(bm[b, h], N, r0, r1)
                s = np.where(keep, s, dtype(-np.inf))                          # :38
                mx = s.max(axis=1, keepdims=True)
                mx_safe = np.where(np.isfinite(mx), mx, dtype(0))
                p = np.exp(s - mx_safe)                                        # :39
                den = p.sum(axis=1, keepdims=True)
                ok = den > 0
                p = p / np.where(ok, den, dtype(1))
                out[b, h, r0:r1] = p @ v[b, h]                                 # :40
                with np.errstate(divide="ignore"):
                    lse[b, h, r0:r1] = np.where(ok, mx_safe + np.log(den), dtype(-np.inf))[:, 0]
    return (out, lse) if return_lse else out


def logsumexp(q, k, block_mask, sm_scale, dtype=np.float32):
    """Natural-log logsumexp over the kept keys of the scaled scores (kernel-test.py:37-38).
    This is NOT the reference kernel's M, which stores only the running maximum in the
    base-2 domain (fa2_custom_mask/fa2_fwd.py:176,191,194-196)."""
    v = np.zeros(np.asarray(k).shape, dtype=dtype)
    return naive_attention(q, k, v, block_mask, sm_scale, dtype=dtype, return_lse=True)[1]


# ----------------------------------------------------------------------------
# tiled online-softmax restatement of the reference kernel
# ----------------------------------------------------------------------------
def tiled_attention(q, k, v, groups, n_list, sm_scale, dtype=np.float32, p_round=None):
    """fa2_custom_mask/fa2_fwd.py:122-206, one python iteration per kept 64x64 tile.

    Returns (O, M, LSE): O as :193, M the reference's stored row maximum in the base-2
    scaled domain (:194-196), LSE = ln2*(m_i + log2(l_i)) (what the upstream kernel
    stores).  Rows of O/M/LSE outside every group stay 0 / -inf.  `p_round` optionally
    rounds P before the second product as :189 does (e.g. np.float16).
    """
    q = np.asarray(q, dtype=dtype); k = np.asarray(k, dtype=dtype); v = np.asarray(v, dtype=dtype)
    B, H, N, D = q.shape
    O = np.zeros((B, H, N, D), dtype=dtype)
    M = np.full((B, H, N), -np.inf, dtype=dtype)
    LSE = np.full((B, H, N), -np.inf, dtype=dtype)
    if groups is None:
        return O, M, LSE
    qk_scale = dtype(sm_scale) * dtype(LOG2E)                     # :150
    for b, h, mb, start, length in np.asarray(groups).tolist():    # :123-128
        rows = slice(mb * TILE, (mb + 1) * TILE)
        qt = q[b, h, rows]                                         # :145
        m_i = np.full(TILE, -np.inf, dtype=dtype)                  # :146
        l_i = np.full(TILE, 1.0, dtype=dtype)                      # :147
        acc = np.zeros((TILE, D), dtype=dtype)                     # :148
        for idx in range(length):                                  # :152
            nblk = int(n_list[start + idx])                        # :153
            cols = slice(nblk * TILE, (nblk + 1) * TILE)
            qk = qt @ k[b, h, cols].T                              # :174-175
            m_ij = np.maximum(m_i, qk.max(axis=1) * qk_scale)      # :176
            p = np.exp2(qk * qk_scale - m_ij[:, None])             # :177-178
            l_ij = p.sum(axis=1)                                   # :179
            alpha = np.exp2(m_i - m_ij)                            # :180
            l_i = l_i * alpha + l_ij                               # :181
            acc = acc * alpha[:, None]                             # :182
            if p_round is not None:
                p = p.astype(p_round).astype(dtype)                # :189
            acc = acc + p @ v[b, h, cols]                          # :190
            m_i = m_ij                                             # :191
        O[b, h, rows] = acc / l_i[:, None]                         # :193
        M[b, h, rows] = m_i                                        # :194-196
        LSE[b, h, rows] = (m_i + np.log2(l_i)) * dtype(np.log(2.0))
    return O, M, LSE


# ----------------------------------------------------------------------------
# backward: the gradient algebra the reference intends
# ----------------------------------------------------------------------------
def attention_backward(q, k, v, block_mask, sm_scale, do, dtype=np.float32, o_stored=None):
    """Gradient of naive_attention w.r.t. q,k,v for upstream gradient `do`.

    Algebra of fa2_custom_mask/fa2_bwd.py: delta = rowsum(O*dO) (:17); P = softmax
    (:57,:117, zero where masked :59-62,:119-123); dV = P^T dO (:67); dP = dO V^T
    (:71,:125); dS = P*(dP - delta) (:72,:126); dK = dS^T Q * sm_scale (:74,:232);
    dQ = dS K * sm_scale (:130 with the host pre-scale fa2_custom_mask.py:110-111, :284).
    Evaluated over full rows (all kept tiles), which is what a correct block-sparse
    backward must equal.  Returns (dq, dk, dv, delta).

    o_stored: the forward's output as it was stored (fp16 / bf16 values).  The reference takes delta from that
    tensor (fa2_custom_mask.py:114-121 hands the saved `o` to _attn_bwd_preprocess, fa2_bwd.py:15-17), not from
    an exact O; the difference only shows where delta is large against dP - delta.  None: the exact O.
    """
    q = np.asarray(q, dtype=dtype); k = np.asarray(k, dtype=dtype); v = np.asarray(v, dtype=dtype)
    do = np.asarray(do, dtype=dtype)
    B, H, N, D = q.shape
    bm = _bcast_mask(block_mask, B, H)
    dq = np.zeros_like(q); dk = np.zeros_like(k); dv = np.zeros_like(v)
    delta = np.zeros((B, H, N), dtype=dtype)
    for b in range(B):
        for h in range(H):
            keep = _keep_rows(bm[b, h], N, 0, N)
            s = (q[b, h] @ k[b, h].T) * dtype(sm_scale)
            s = np.where(keep, s, dtype(-np.inf))
            mx = s.max(axis=1, keepdims=True)
            mx = np.where(np.isfinite(mx), mx, dtype(0))
            p = np.exp(s - mx)
            den = p.sum(axis=1, keepdims=True)
            p = p / np.where(den > 0, den, dtype(1))
            o = p @ v[b, h] if o_stored is None else np.asarray(o_stored, dtype=dtype)[b, h]
            dl = (o * do[b, h]).sum(axis=1)                        # fa2_bwd.py:17
            dv[b, h] = p.T @ do[b, h]                              # :67
            dp = do[b, h] @ v[b, h].T                              # :71
            ds = p * (dp - dl[:, None])                            # :72
            dk[b, h] = (ds.T @ q[b, h]) * dtype(sm_scale)          # :74,:232
            dq[b, h] = (ds @ k[b, h]) * dtype(sm_scale)            # :130,:284
            delta[b, h] = dl
    return dq, dk, dv, delta


# ----------------------------------------------------------------------------
# head-wise token reorder (the steps either side of attention in the caller)
# ----------------------------------------------------------------------------
PERMUTATIONS = np.array([[0, 1, 2], [0, 2, 1], [1, 2, 0],
                         [1, 0, 2], [2, 1, 0], [2, 0, 1]], dtype=np.int32)      # functional.py:23-26
PERMUTATIONS_INV = np.array([[0, 1, 2], [0, 2, 1], [2, 0, 1],
                             [1, 0, 2], [2, 1, 0], [1, 2, 0]], dtype=np.int32)  # functional.py:69-76


def _new_token(f, h_, w, dims, p):
    """fa2_custom_mask/permute.py:41-52: new_t = c0*(d1*d2) + c1*d2 + c2."""
    coords = (f, h_, w)
    c0, c1, c2 = coords[p[0]], coords[p[1]], coords[p[2]]
    d1, d2 = dims[p[1]], dims[p[2]]
    return c0 * (d1 * d2) + c1 * d2 + c2


def reorder(x, permute_orders, F, H, W):
    """fa2_custom_mask/permute.py:5-58: out[b,hd,new_t,:] = in[b,hd,t,:] per head, scalar loops."""
    x = np.asarray(x)
    BS, NH, T, D = x.shape
    assert T == F * H * W                                       # functional.py:7
    out = np.empty_like(x)
    for hd in range(NH):
        p = [int(v) for v in permute_orders[hd]]                 # permute.py:33-35
        for t in range(T):
            f, t_ = divmod(t, H * W)                             # :27-30
            h_, w = divmod(t_, W)
            nt = _new_token(f, h_, w, (F, H, W), p)
            out[:, hd, nt, :] = x[:, hd, t, :]                   # :54-58
    return out


def inv_reorder(x, permute_orders, inv_permute_orders, F, H, W):
    """fa2_custom_mask/permute.py:60-126: decode t in the permuted dims (:77-98), then
    re-encode with the inverse order (:101-120)."""
    x = np.asarray(x)
    BS, NH, T, D = x.shape
    assert T == F * H * W                                       # functional.py:48
    out = np.empty_like(x)
    dims0 = (F, H, W)
    for hd in range(NH):
        fp = [int(v) for v in permute_orders[hd]]                # :77-79
        dims = (dims0[fp[0]], dims0[fp[1]], dims0[fp[2]])        # :81-87
        p = [int(v) for v in inv_permute_orders[hd]]             # :101-103
        for t in range(T):
            f, t_ = divmod(t, dims[1] * dims[2])                 # :90-95
            h_, w = divmod(t_, dims[2])
            nt = _new_token(f, h_, w, dims, p)
            out[:, hd, nt, :] = x[:, hd, t, :]                   # :122-126
    return out
