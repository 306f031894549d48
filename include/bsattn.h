/*
 * bsattn.h - C ABI of libbsattn.so: block-sparse FlashAttention-2 for AMD MI355X (gfx950).
 *
 * This is the boundary a replacement for the reference's device layer binds to.  The
 * reference has no native FFI of its own (its device code is Triton JIT launched from
 * Python); each entry point below names the reference Python/Triton interface it
 * replaces, with paths relative to the reference repository root.
 *
 * Conventions
 *   - plain C types only; every function returns 0 (BSATTN_OK) or a negative error code;
 *   - all argument validation happens before any device work, so error paths can be
 *     exercised on a host without a GPU;
 *   - all buffers are caller-owned device memory (raw pointers, e.g. tensor.data_ptr());
 *     the library never allocates or frees device memory: scratch is passed in as a
 *     workspace whose size is queried first;
 *   - every call only enqueues work on `stream` (a hipStream_t passed as void*, NULL = the
 *     default stream) and never synchronises;
 *   - strides are in elements, int64; tiles are fixed 64x64 (reference:
 *     fa2_custom_mask/fa2_fwd.py:13-14).
 */
#ifndef BSATTN_H_
#define BSATTN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BSATTN_TILE 64

/* error codes */
#define BSATTN_OK 0
#define BSATTN_ERR_NULL (-1)       /* a required pointer is NULL */
#define BSATTN_ERR_SHAPE (-2)      /* non-positive size, N not a multiple of 64, bad broadcast */
#define BSATTN_ERR_DTYPE (-3)      /* unknown dtype code */
#define BSATTN_ERR_HEAD_DIM (-4)   /* head dimension not in {64, 128, 256} */
#define BSATTN_ERR_STRIDE (-5)     /* innermost stride != 1 or rows not 16-byte aligned */
#define BSATTN_ERR_WORKSPACE (-6)  /* workspace NULL or too small */
#define BSATTN_ERR_LAUNCH (-7)     /* the HIP runtime refused a launch */
#define BSATTN_ERR_RANGE (-8)      /* a size exceeds what 32-bit indices can address */
#define BSATTN_ERR_STATIC_LIMIT (-9) /* bsattn_fwd_static: the shape needs more scratch memory than
                                        BSATTN_STATIC_SCRATCH_BYTES */

/* dtype codes */
#define BSATTN_F16 0
#define BSATTN_BF16 1
#define BSATTN_F32 2 /* outputs only */

/* ABI version of the library, major * 100 + minor.  The major number changes whenever an entry point's
 * argument list changes or an entry point goes away; a caller built against this header checks
 * bsattn_version() / 100 == BSATTN_ABI_VERSION / 100 before its first other call.
 *   100: first layout.
 *   200: bsattn_bwd and bsattn_bwd_elementwise take dq_strides, dk_strides, dv_strides after
 *        do_strides; the entry points of the forward over quads of row blocks are gone. */
#define BSATTN_ABI_VERSION 200
int bsattn_version(void);
/* Process-wide switch (default off), returns the previous setting.  On: the forward's result
 * depends on nothing but its inputs and the device (two runs give the same bits).  Off: the
 * tiles of a row block are handed to the wavefronts of a workgroup as they become free, which
 * is faster and changes the order of summation, i.e. the last bits, from run to run.  The
 * backward and the preprocessing are deterministic either way.  No counterpart in the
 * reference (Triton's kernels there are deterministic by construction). */
int bsattn_set_deterministic(int on);
/* Static string for an error code; never freed by the caller. */
const char* bsattn_strerror(int code);

/* ------------------------------------------------------------------------------------
 * Mask preprocessing (integer work, bit-exact).
 * Replaces build_groups_from_block_mask, fa2_custom_mask/fa2_custom_mask.py:15-38, which
 * the reference runs as a Python triple loop with one torch.nonzero + host sync per row.
 * ---------------------------------------------------------------------------------- */

/* Reduce an elementwise mask [Bm,Hm,N,N] (bool bytes, innermost stride 1, row stride a
 * multiple of 16 and a 16-byte aligned base) to a block mask [Bm,Hm,N/64,N/64]
 * (contiguous bool bytes): a tile is kept iff any of its 64x64 elements is set.  This is
 * the inverse of the expansion at kernel-test.py:18 for tile-constant masks. */
int bsattn_reduce_dense_mask(const uint8_t* dense, int Bm, int Hm, int N,
                             int64_t sb, int64_t sh, int64_t sm,
                             uint8_t* block_out, void* stream);

/* Bytes of workspace bsattn_block_mask_to_lists needs for Bm*Hm*nb rows (4-byte aligned; its contents
 * on entry do not matter). */
int bsattn_mask_lists_workspace(int Bm, int Hm, int nb, size_t* bytes);

/* Block mask [Bm,Hm,nb,nb] (bool bytes, arbitrary element strides; pass the row/column
 * strides swapped to obtain the column lists a backward pass needs) -> kept-tile lists:
 *   row_ptr  int32 [Bm*Hm*nb + 1]  exclusive prefix sum of kept tiles per row
 *   col_idx  int32 [capacity Bm*Hm*nb*nb]  ascending kept column tiles, row after row
 *                                  (identical to the reference's n_list)
 *   groups   int32 [capacity Bm*Hm*nb, 5] or NULL: the reference's (b,h,m_block,start,len)
 *                                  rows with empty rows omitted (fa2_custom_mask.py:29-33)
 *   counts   int32 [2]: G (rows of `groups`) and T (kept tiles); (0,0) corresponds to the
 *                                  reference returning (None, None) (fa2_custom_mask.py:34-35)
 */
int bsattn_block_mask_to_lists(const uint8_t* block, int Bm, int Hm, int nb,
                               int64_t sb, int64_t sh, int64_t sm, int64_t sn,
                               int32_t* row_ptr, int32_t* col_idx, int32_t* groups,
                               int32_t* counts, void* workspace, size_t workspace_bytes,
                               void* stream);

/* ------------------------------------------------------------------------------------
 * Elementwise masks (exact semantics inside partly set tiles: the naive masked_fill(-inf)
 * of kernel-test.py:38, which the reference's dead elementwise loop fa2_fwd.py:67-73 and
 * its backward fa2_bwd.py:59-62,119-123 intend).  For every entry t of the kept-tile lists
 * of the reduced mask: tile_partial[t] = 1 if the tile is only partly set, and
 * tile_bits[64 t + r] = the 64 bools of row r of the tile (bit c = column c).
 * dense: bool bytes [Bm,Hm,N,N] with element strides sb, sh, sm (rows), sn (columns);
 * row_ptr/col_idx: lists of the reduced mask as made by bsattn_block_mask_to_lists.
 * Passing the lists of the transposed block mask together with sm and sn swapped gives
 * the per-key words the dK/dV pass uses.  tile_partial: nb*nb*Bm*Hm bytes capacity,
 * tile_bits: 64 times as many 64-bit words.  sn == 1 needs 4-byte aligned rows.
 * ---------------------------------------------------------------------------------- */
int bsattn_pack_mask_tiles(const uint8_t* dense, int Bm, int Hm, int N, int64_t sb, int64_t sh,
                           int64_t sm, int64_t sn, const int32_t* row_ptr, const int32_t* col_idx,
                           uint8_t* tile_partial, uint64_t* tile_bits, void* stream);

/* The same words in one pass over the mask, for callers that start from the elementwise mask itself: the
 * block mask (as bsattn_reduce_dense_mask gives it), and for every tile of the grid that has a set element
 * its "partly set" flag and its 64 words, at the tile's grid position
 * g = (mask head * nb + row block) * nb + column block: grid_partial[g], grid_bits[64 g + r] (tiles without
 * a set element get grid_partial = 0 and their words are left unwritten).  dense: innermost stride 1, the
 * other strides multiples of 16 and a 16-byte aligned base; grid_partial: Bm*Hm*nb*nb bytes, grid_bits: 64
 * times as many 64-bit words.  bsattn_gather_mask_tiles then moves the words of the kept tiles to their
 * list positions (the format bsattn_fwd_elementwise / bsattn_bwd_elementwise take): with the row lists and
 * transposed = 0 as they are, with the column lists (bsattn_block_mask_to_lists with the block mask's row
 * and column strides swapped) and transposed = 1 as the per-key words of the dK/dV pass.  The mask is read
 * once for all of it.  Same semantics as bsattn_pack_mask_tiles (kernel-test.py:38). */
int bsattn_reduce_pack_dense_mask(const uint8_t* dense, int Bm, int Hm, int N, int64_t sb, int64_t sh,
                                  int64_t sm, uint8_t* block_out, uint8_t* grid_partial,
                                  uint64_t* grid_bits, void* stream);
int bsattn_gather_mask_tiles(const uint8_t* grid_partial, const uint64_t* grid_bits, int Bm, int Hm,
                             int nb, int transposed, const int32_t* row_ptr, const int32_t* col_idx,
                             uint8_t* tile_partial, uint64_t* tile_bits, void* stream);

/* Sequence lengths N that are not a multiple of 64 (unsupported by the reference, whose block
 * pointers assume whole tiles: fa2_custom_mask/fa2_fwd.py:137-172): the caller pads q, k, v
 * with zero rows to nb*64 tokens and masks the padding keys through the elementwise entry
 * points.  This fills tile_partial / tile_bits (same format and capacity as
 * bsattn_pack_mask_tiles) for the lists of a block mask [Bm,Hm,nb,nb] whose last column block
 * holds only valid_last (1..64) real keys: every tile is completely set except those of the
 * last column block, which keep their first valid_last keys.  transposed != 0: row_ptr /
 * col_idx are the column lists (the words the dK/dV pass uses). */
int bsattn_tail_mask_tiles(int Bm, int Hm, int nb, int valid_last, int transposed,
                           const int32_t* row_ptr, const int32_t* col_idx, uint8_t* tile_partial,
                           uint64_t* tile_bits, void* stream);

/* ------------------------------------------------------------------------------------
 * Forward.  Replaces the launch of _attn_fwd (fa2_custom_mask/fa2_fwd.py:108-206) from
 * _attention.forward (fa2_custom_mask/fa2_custom_mask.py:69-87).
 * ---------------------------------------------------------------------------------- */

/* Bytes of workspace bsattn_fwd needs (partial results of row blocks whose kept-tile list
 * is split over several wavefronts). */
int bsattn_fwd_workspace(int B, int H, int N, int D, size_t* bytes);

/* q,k,v: [B,H,N,D] fp16/bf16 (dtype), strides[4] each, innermost stride 1.
 * o:     [B,H,N,D] of out_dtype (dtype itself or BSATTN_F32), strides o_strides.
 * lse:   fp32 [B,H,N] contiguous or NULL: natural-log logsumexp of the kept scaled scores.
 *        (The reference's M output, fa2_fwd.py:194-196, is the running maximum only and is
 *        not reproduced.)
 * row_ptr/col_idx: lists from bsattn_block_mask_to_lists for a [Bm,Hm,nb,nb] mask,
 *        Bm in {1,B}, Hm in {1,H} (1 = shared across that axis).
 * Row blocks without a kept tile get O = 0 and lse = -inf (the reference leaves them
 * unwritten: fa2_custom_mask.py:29-30,59).
 * A row block whose kept tiles are split over several workgroups is finished by the workgroup
 * that completes its share last (parts and one counter per row block live in the workspace):
 * no workgroup ever waits for another, so the call completes whatever else runs on the GPU
 * and however many workgroups are resident at a time.  The workspace (16-byte aligned, else
 * BSATTN_ERR_STRIDE: it holds 64-bit counters behind the parts) needs no initialisation
 * and may be reused by the next call on the same stream; two calls that overlap in time need
 * two workspaces.
 * Memory ordering of that hand-off.  A holder of a part writes it with device-scope stores (they
 * are served by the memory all compute units share, never by a cache only some of them see), waits
 * until every one of them has been acknowledged (s_waitcnt vmcnt(0) in each wavefront, then the
 * workgroup barrier), and only then does one thread count the part in with a compare-and-swap on
 * the row block's counter.  The workgroup that finds all other parts counted reads them with
 * device-scope loads issued after its compare-and-swap has returned (the value is passed through
 * LDS and a barrier to the other wavefronts, so no load of a part can be issued before it).  Each
 * part was complete in shared memory before its count became visible, and the reader's loads
 * cannot be served from a stale cache line, so the counter update itself is relaxed: release /
 * acquire order on it would add a write-back and an invalidation of a whole L2 for accesses that
 * are already ordered, measured at 9 us per launch (N = 17536, one head, keep 0.1: 31 -> 41 us).
 * A counter holds (launch mark << 16 | parts counted): contents left by earlier launches carry
 * another mark and read as zero, and the last arriver puts the counter back to zero. */
int bsattn_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
               const int32_t* row_ptr, const int32_t* col_idx, int Bm, int Hm,
               int B, int H, int N, int D, int dtype, int out_dtype, float sm_scale,
               const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
               const int64_t* o_strides, void* workspace, size_t workspace_bytes,
               void* stream);

/* The reference's whole forward call in one: _attention.forward (fa2_custom_mask/fa2_custom_mask.py:43-94) builds
 * the lists of the block mask (:48) and launches _attn_fwd on them (:77-87).  This entry point enqueues
 * bsattn_block_mask_to_lists (without `groups`) and bsattn_fwd on `stream` from one host call, for callers
 * whose mask changes from call to call; row_ptr, col_idx (capacities as for bsattn_block_mask_to_lists) and
 * counts are left filled and may be handed to later bsattn_fwd / bsattn_bwd calls for the same mask.
 * mask_strides: the four element strides of the bool [Bm,Hm,nb,nb] mask, nb = N / 64 (0 or any value for
 * dimensions of size 1).  One workspace of bsattn_fwd_block_mask_workspace bytes (16-byte aligned) serves both
 * steps.  All arguments are checked before the first launch. */
int bsattn_fwd_block_mask_workspace(int Bm, int Hm, int B, int H, int N, int D, size_t* bytes);
int bsattn_fwd_block_mask(const void* q, const void* k, const void* v, void* o, float* lse,
                          const uint8_t* block, const int64_t* mask_strides, int Bm, int Hm,
                          int32_t* row_ptr, int32_t* col_idx, int32_t* counts,
                          int B, int H, int N, int D, int dtype, int out_dtype, float sm_scale,
                          const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                          const int64_t* o_strides, void* workspace, size_t workspace_bytes,
                          void* stream);

/* Forward that allocates nothing and needs no workspace argument.  It has no counterpart in the
 * reference; it is for callers that cannot allocate device memory around the call: code under HIP
 * graph capture, tight serving loops, harnesses that forbid allocation.  Same arguments, results and
 * kernels as bsattn_fwd, with the workspace replaced by a device array of
 * BSATTN_STATIC_SCRATCH_BYTES that is part of the library (every GPU the library runs on holds its
 * own copy until the process ends).  Shapes whose parts and flags (the memory
 * bsattn_fwd's kernels use out of its workspace) exceed that size are
 * rejected with BSATTN_ERR_STATIC_LIMIT before any device work.  All calls on one GPU share the
 * array: two calls that overlap in time on the same GPU (different streams or threads) race and
 * must be serialised by the caller; calls on one stream are ordered and safe.  Nothing has to be
 * cleared between calls (stale contents are told apart by a per-launch number).  The first call on
 * a device looks up the array's address (no allocation, but not capturable: make one call before
 * capturing). */
#define BSATTN_STATIC_SCRATCH_BYTES (32u << 20)
int bsattn_fwd_static(const void* q, const void* k, const void* v, void* o, float* lse,
                      const int32_t* row_ptr, const int32_t* col_idx, int Bm, int Hm,
                      int B, int H, int N, int D, int dtype, int out_dtype, float sm_scale,
                      const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                      const int64_t* o_strides, void* stream);

/* ------------------------------------------------------------------------------------
 * Forward with an elementwise mask: as bsattn_fwd, and inside the kept tiles flagged in
 * tile_partial the scores of unset elements are -inf (kernel-test.py:38; the semantics
 * the reference's unused inner loop fa2_fwd.py:67-73 intends).  tile_partial / tile_bits
 * as made by bsattn_pack_mask_tiles for the same lists.  Query rows without any set
 * element give O = 0, lse = -inf.
 * ---------------------------------------------------------------------------------- */
int bsattn_fwd_elementwise(const void* q, const void* k, const void* v, void* o, float* lse,
                           const int32_t* row_ptr, const int32_t* col_idx,
                           const uint8_t* tile_partial, const uint64_t* tile_bits, int Bm, int Hm,
                           int B, int H, int N, int D, int dtype, int out_dtype, float sm_scale,
                           const int64_t* q_strides, const int64_t* k_strides,
                           const int64_t* v_strides, const int64_t* o_strides, void* workspace,
                           size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------
 * Backward.  Replaces _attn_bwd_preprocess and _attn_bwd (fa2_custom_mask/fa2_bwd.py:5-19,
 * 140-285) as launched from _attention.backward (fa2_custom_mask/fa2_custom_mask.py:97-155).
 * The gradient algebra is the reference's (fa2_bwd.py:17,57-74,117-130,232,284) evaluated
 * over exactly the kept tiles.
 * ---------------------------------------------------------------------------------- */

/* Bytes of workspace bsattn_bwd needs: delta = rowsum(O * dO), and for launches with few row
 * blocks the fp32 parts of dQ, dK, dV of row / column lists walked by several workgroups.
 * Depends on the shape and on the number of compute units of the current device.  The workspace
 * must be 16-byte aligned (BSATTN_ERR_STRIDE otherwise). */
int bsattn_bwd_workspace(int B, int H, int N, int D, size_t* bytes);

/* q,k,v,o,d_o: [B,H,N,D] fp16/bf16 with their own strides; lse from bsattn_fwd.
 * dq,dk,dv: [B,H,N,D] of out_dtype with strides dq_strides, dk_strides, dv_strides (innermost 1;
 *        NULL: no gaps), e.g. the three slices of one packed [B,N,3,H,D] gradient buffer, as the
 *        reference's torch.empty_like(q) gives for such inputs (fa2_custom_mask.py:101-103).
 * row_ptr/col_idx: row lists; col_ptr/row_idx: column lists (the same call with the mask's
 * row and column strides swapped). */
int bsattn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
               const float* lse, void* dq, void* dk, void* dv,
               const int32_t* row_ptr, const int32_t* col_idx,
               const int32_t* col_ptr, const int32_t* row_idx, int Bm, int Hm,
               int B, int H, int N, int D, int dtype, int out_dtype, float sm_scale,
               const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
               const int64_t* o_strides, const int64_t* do_strides,
               const int64_t* dq_strides, const int64_t* dk_strides, const int64_t* dv_strides,
               void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------
 * Backward with an elementwise mask: as bsattn_bwd, with P = 0 at unset elements (the
 * zeroing fa2_bwd.py:59-62,119-123 intends).  tile_bits_rows: words of the row lists
 * (bsattn_pack_mask_tiles on row_ptr/col_idx), tile_bits_cols: words of the column lists
 * (the same call on col_ptr/row_idx with the mask's row and column strides swapped).
 * Rows whose lse is -inf get zero gradients.
 * ---------------------------------------------------------------------------------- */
int bsattn_bwd_elementwise(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                           const float* lse, void* dq, void* dk, void* dv, const int32_t* row_ptr,
                           const int32_t* col_idx, const int32_t* col_ptr, const int32_t* row_idx,
                           const uint64_t* tile_bits_rows, const uint64_t* tile_bits_cols,
                           int Bm, int Hm, int B, int H, int N, int D, int dtype, int out_dtype,
                           float sm_scale, const int64_t* q_strides, const int64_t* k_strides,
                           const int64_t* v_strides, const int64_t* o_strides,
                           const int64_t* do_strides, const int64_t* dq_strides,
                           const int64_t* dk_strides, const int64_t* dv_strides, void* workspace,
                           size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------
 * Head-wise token reorder.  Replaces reorder_kernel / inv_reorder_kernel
 * (fa2_custom_mask/permute.py:5-58, 60-126) as launched from apply_head_wise_reorder /
 * apply_inv_reorder (fa2_custom_mask/functional.py:5-20, 46-62).
 * x,out: [BS,NH,F*Hh*W,D] contiguous, elem_bytes per element (row bytes a multiple of 4);
 * orders: int32 [NH,3] device memory; inv_orders: int32 [NH,3] or NULL (forward reorder).
 * out[b,h,new_t,:] = x[b,h,t,:] with new_t as permute.py:45-52.
 * ---------------------------------------------------------------------------------- */
int bsattn_reorder(const void* x, void* out, int BS, int NH, int F, int Hh, int W, int D,
                   int elem_bytes, const int32_t* orders, const int32_t* inv_orders,
                   void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BSATTN_H_ */
