// extern "C" entry points: argument validation first, then launches.  No device memory is
// allocated or freed here and nothing synchronises; every error is detected before the
// first launch so that the error paths behave the same on a host without a GPU.
#include "common.h"

using namespace bsattn;

extern "C" {

int bsattn_version(void) { return BSATTN_VERSION; }

int bsattn_set_deterministic(int on) { return set_deterministic(on); }

const char* bsattn_strerror(int code) {
  switch (code) {
    case BSATTN_OK: return "ok";
    case BSATTN_ERR_NULL: return "a required pointer is NULL";
    case BSATTN_ERR_SHAPE: return "bad shape: sizes must be positive, N a multiple of 64, mask batch/head sizes 1 or equal to B/H";
    case BSATTN_ERR_DTYPE: return "unsupported dtype code";
    case BSATTN_ERR_HEAD_DIM: return "head dimension must be 64, 128 or 256";
    case BSATTN_ERR_STRIDE: return "innermost stride must be 1 and rows 16-byte aligned";
    case BSATTN_ERR_WORKSPACE: return "workspace missing or too small";
    case BSATTN_ERR_LAUNCH: return "HIP launch failed";
    case BSATTN_ERR_RANGE: return "size exceeds 32-bit index range";
    case BSATTN_ERR_STATIC_LIMIT: return "shape needs more scratch memory than the library's static buffer holds";
    default: return "unknown error code";
  }
}

int bsattn_reduce_dense_mask(const uint8_t* dense, int Bm, int Hm, int N, int64_t sb, int64_t sh,
                             int64_t sm, uint8_t* block_out, void* stream) {
  if (dense == nullptr || block_out == nullptr) return BSATTN_ERR_NULL;
  if (Bm <= 0 || Hm <= 0 || N <= 0 || N % BSATTN_TILE != 0) return BSATTN_ERR_SHAPE;
  if ((int64_t)Bm * Hm > 65535) return BSATTN_ERR_RANGE;
  if (sm % 16 != 0 || sb % 16 != 0 || sh % 16 != 0 || ((uintptr_t)dense & 15) != 0) return BSATTN_ERR_STRIDE;
  return launch_reduce_dense_mask(dense, Bm, Hm, N, sb, sh, sm, block_out, (hipStream_t)stream);
}

int bsattn_mask_lists_workspace(int Bm, int Hm, int nb, size_t* bytes) {
  if (bytes == nullptr) return BSATTN_ERR_NULL;
  if (Bm <= 0 || Hm <= 0 || nb <= 0) return BSATTN_ERR_SHAPE;
  if ((int64_t)Bm * Hm * nb * nb > 0x7fffffffLL) return BSATTN_ERR_RANGE;
  *bytes = (size_t)Bm * Hm * nb * 2 * sizeof(int32_t);     // per row: count, position in `groups`
  return BSATTN_OK;
}

int bsattn_block_mask_to_lists(const uint8_t* block, int Bm, int Hm, int nb, int64_t sb, int64_t sh,
                               int64_t sm, int64_t sn, int32_t* row_ptr, int32_t* col_idx,
                               int32_t* groups, int32_t* counts, void* workspace,
                               size_t workspace_bytes, void* stream) {
  if (block == nullptr || row_ptr == nullptr || col_idx == nullptr || counts == nullptr) return BSATTN_ERR_NULL;
  size_t need = 0;
  const int rc = bsattn_mask_lists_workspace(Bm, Hm, nb, &need);
  if (rc != BSATTN_OK) return rc;
  if (workspace == nullptr || workspace_bytes < need) return BSATTN_ERR_WORKSPACE;
  if (((uintptr_t)workspace & 3) != 0) return BSATTN_ERR_STRIDE;
  return launch_block_mask_to_lists(block, Bm, Hm, nb, sb, sh, sm, sn, row_ptr, col_idx, groups, counts,
                                    (int32_t*)workspace, (hipStream_t)stream);
}

int bsattn_pack_mask_tiles(const uint8_t* dense, int Bm, int Hm, int N, int64_t sb, int64_t sh, int64_t sm,
                           int64_t sn, const int32_t* row_ptr, const int32_t* col_idx, uint8_t* tile_partial,
                           uint64_t* tile_bits, void* stream) {
  if (dense == nullptr || row_ptr == nullptr || col_idx == nullptr || tile_partial == nullptr || tile_bits == nullptr)
    return BSATTN_ERR_NULL;
  if (Bm <= 0 || Hm <= 0 || N <= 0 || N % BSATTN_TILE != 0) return BSATTN_ERR_SHAPE;
  if ((int64_t)Bm * Hm > 65535) return BSATTN_ERR_RANGE;
  if (sn == 1 && ((sm % 4) != 0 || (sb % 4) != 0 || (sh % 4) != 0 || ((uintptr_t)dense & 3) != 0)) return BSATTN_ERR_STRIDE;
  return launch_pack_tiles(dense, Bm, Hm, N / BSATTN_TILE, sb, sh, sm, sn, row_ptr, col_idx, tile_partial,
                           (unsigned long long*)tile_bits, (hipStream_t)stream);
}

int bsattn_reduce_pack_dense_mask(const uint8_t* dense, int Bm, int Hm, int N, int64_t sb, int64_t sh, int64_t sm,
                                  uint8_t* block_out, uint8_t* grid_partial, uint64_t* grid_bits, void* stream) {
  if (dense == nullptr || block_out == nullptr || grid_partial == nullptr || grid_bits == nullptr) return BSATTN_ERR_NULL;
  if (Bm <= 0 || Hm <= 0 || N <= 0 || N % BSATTN_TILE != 0) return BSATTN_ERR_SHAPE;
  if ((int64_t)Bm * Hm > 65535) return BSATTN_ERR_RANGE;
  if ((sm % 16) != 0 || (sb % 16) != 0 || (sh % 16) != 0 || ((uintptr_t)dense & 15) != 0 || ((uintptr_t)grid_bits & 7) != 0)
    return BSATTN_ERR_STRIDE;
  return launch_reduce_pack(dense, Bm, Hm, N, sb, sh, sm, block_out, grid_partial, (unsigned long long*)grid_bits,
                            (hipStream_t)stream);
}

int bsattn_gather_mask_tiles(const uint8_t* grid_partial, const uint64_t* grid_bits, int Bm, int Hm, int nb,
                             int transposed, const int32_t* row_ptr, const int32_t* col_idx, uint8_t* tile_partial,
                             uint64_t* tile_bits, void* stream) {
  if (grid_partial == nullptr || grid_bits == nullptr || row_ptr == nullptr || col_idx == nullptr ||
      tile_partial == nullptr || tile_bits == nullptr)
    return BSATTN_ERR_NULL;
  if (Bm <= 0 || Hm <= 0 || nb <= 0) return BSATTN_ERR_SHAPE;
  if ((int64_t)Bm * Hm > 65535 || (int64_t)Bm * Hm * nb * nb > 0x7fffffffLL) return BSATTN_ERR_RANGE;
  if ((((uintptr_t)grid_bits | (uintptr_t)tile_bits) & 7) != 0) return BSATTN_ERR_STRIDE;
  return launch_gather_tiles(grid_partial, (const unsigned long long*)grid_bits, Bm, Hm, nb, transposed != 0, row_ptr, col_idx,
                             tile_partial, (unsigned long long*)tile_bits, (hipStream_t)stream);
}

int bsattn_tail_mask_tiles(int Bm, int Hm, int nb, int valid_last, int transposed, const int32_t* row_ptr,
                           const int32_t* col_idx, uint8_t* tile_partial, uint64_t* tile_bits, void* stream) {
  if (row_ptr == nullptr || col_idx == nullptr || tile_partial == nullptr || tile_bits == nullptr) return BSATTN_ERR_NULL;
  if (Bm <= 0 || Hm <= 0 || nb <= 0 || valid_last < 1 || valid_last > BSATTN_TILE) return BSATTN_ERR_SHAPE;
  if ((int64_t)Bm * Hm * nb > 0x7fffffff) return BSATTN_ERR_RANGE;
  return launch_tail_tiles(Bm, Hm, nb, valid_last, transposed != 0, row_ptr, col_idx, tile_partial,
                           (unsigned long long*)tile_bits, (hipStream_t)stream);
}

static int check_attn(int Bm, int Hm, int B, int H, int N, int D, int dtype, int out_dtype) {
  if (B <= 0 || H <= 0 || N <= 0 || N % BSATTN_TILE != 0) return BSATTN_ERR_SHAPE;
  if (!((Bm == 1 || Bm == B) && (Hm == 1 || Hm == H))) return BSATTN_ERR_SHAPE;
  if (D != 64 && D != 128 && D != 256) return BSATTN_ERR_HEAD_DIM;
  if (dtype != BSATTN_F16 && dtype != BSATTN_BF16) return BSATTN_ERR_DTYPE;
  if (out_dtype != dtype && out_dtype != BSATTN_F32) return BSATTN_ERR_DTYPE;
  if ((int64_t)B * H > 65535) return BSATTN_ERR_RANGE;
  const int64_t nb = N / BSATTN_TILE;
  if ((int64_t)Bm * Hm * nb * nb > 0x7fffffffLL) return BSATTN_ERR_RANGE;
  return BSATTN_OK;
}

static int check_strides(const int64_t* s, int elem_bytes, const void* base) {
  if (s == nullptr) return BSATTN_ERR_NULL;
  if (s[3] != 1) return BSATTN_ERR_STRIDE;
  for (int i = 0; i < 3; ++i)
    if ((s[i] * elem_bytes) % 16 != 0) return BSATTN_ERR_STRIDE;
  if (((uintptr_t)base & 15) != 0) return BSATTN_ERR_STRIDE;
  return BSATTN_OK;
}

int bsattn_fwd_workspace(int B, int H, int N, int D, size_t* bytes) {
  if (bytes == nullptr) return BSATTN_ERR_NULL;
  const int rc = check_attn(1, 1, B, H, N, D, BSATTN_F16, BSATTN_F16);
  if (rc != BSATTN_OK) return rc;
  *bytes = fwd_workspace_bytes(B, H, N, D);
  return BSATTN_OK;
}

// Everything bsattn_fwd and its variants check before the workspace question.
static int fwd_check(const void* q, const void* k, const void* v, void* o, const int32_t* row_ptr,
                     const int32_t* col_idx, int Bm, int Hm, int B, int H, int N, int D, int dtype,
                     int out_dtype, const int64_t* q_strides, const int64_t* k_strides,
                     const int64_t* v_strides, const int64_t* o_strides) {
  if (q == nullptr || k == nullptr || v == nullptr || o == nullptr || row_ptr == nullptr || col_idx == nullptr)
    return BSATTN_ERR_NULL;
  int rc = check_attn(Bm, Hm, B, H, N, D, dtype, out_dtype);
  if (rc != BSATTN_OK) return rc;
  if ((rc = check_strides(q_strides, 2, q)) != BSATTN_OK) return rc;
  if ((rc = check_strides(k_strides, 2, k)) != BSATTN_OK) return rc;
  if ((rc = check_strides(v_strides, 2, v)) != BSATTN_OK) return rc;
  return check_strides(o_strides, out_dtype == BSATTN_F32 ? 4 : 2, o);
}

static int fwd_common(const void* q, const void* k, const void* v, void* o, float* lse,
                      const int32_t* row_ptr, const int32_t* col_idx, const uint8_t* tile_partial,
                      const uint64_t* tile_bits, int Bm, int Hm, int B, int H, int N,
                      int D, int dtype, int out_dtype, float sm_scale, const int64_t* q_strides,
                      const int64_t* k_strides, const int64_t* v_strides, const int64_t* o_strides,
                      void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = fwd_check(q, k, v, o, row_ptr, col_idx, Bm, Hm, B, H, N, D, dtype, out_dtype, q_strides, k_strides,
                           v_strides, o_strides);
  if (rc != BSATTN_OK) return rc;
  if (workspace == nullptr || workspace_bytes < coop_workspace_bytes(B, H, N, D)) return BSATTN_ERR_WORKSPACE;
  if (((uintptr_t)workspace & 15) != 0) return BSATTN_ERR_STRIDE;
  AttnShape s;
  s.B = B; s.H = H; s.N = N; s.D = D; s.Bm = Bm; s.Hm = Hm; s.dtype = dtype; s.out_dtype = out_dtype;
  s.sm_scale = sm_scale;
  for (int i = 0; i < 3; ++i) { s.qs[i] = q_strides[i]; s.ks[i] = k_strides[i]; s.vs[i] = v_strides[i]; s.os[i] = o_strides[i]; s.dos[i] = 0; }
  return launch_fwd(q, k, v, o, lse, row_ptr, col_idx, tile_partial, tile_bits, s, workspace, (hipStream_t)stream);
}

int bsattn_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
               const int32_t* row_ptr, const int32_t* col_idx, int Bm, int Hm, int B, int H, int N,
               int D, int dtype, int out_dtype, float sm_scale, const int64_t* q_strides,
               const int64_t* k_strides, const int64_t* v_strides, const int64_t* o_strides,
               void* workspace, size_t workspace_bytes, void* stream) {
  return fwd_common(q, k, v, o, lse, row_ptr, col_idx, nullptr, nullptr, Bm, Hm, B, H, N, D, dtype, out_dtype,
                    sm_scale, q_strides, k_strides, v_strides, o_strides, workspace, workspace_bytes, stream);
}

// the lists part of bsattn_fwd_block_mask's workspace, rounded up so that the forward's part stays aligned
static size_t lists_part_bytes(int Bm, int Hm, int nb) {
  return (((size_t)Bm * Hm * nb * 2 * sizeof(int32_t)) + 255) & ~(size_t)255;
}

int bsattn_fwd_block_mask_workspace(int Bm, int Hm, int B, int H, int N, int D, size_t* bytes) {
  if (bytes == nullptr) return BSATTN_ERR_NULL;
  int rc = check_attn(Bm, Hm, B, H, N, D, BSATTN_F16, BSATTN_F16);
  if (rc != BSATTN_OK) return rc;
  size_t lists = 0;
  if ((rc = bsattn_mask_lists_workspace(Bm, Hm, N / BSATTN_TILE, &lists)) != BSATTN_OK) return rc;
  *bytes = lists_part_bytes(Bm, Hm, N / BSATTN_TILE) + fwd_workspace_bytes(B, H, N, D);
  return BSATTN_OK;
}

int bsattn_fwd_block_mask(const void* q, const void* k, const void* v, void* o, float* lse, const uint8_t* block,
                          const int64_t* mask_strides, int Bm, int Hm, int32_t* row_ptr, int32_t* col_idx,
                          int32_t* counts, int B, int H, int N, int D, int dtype, int out_dtype, float sm_scale,
                          const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                          const int64_t* o_strides, void* workspace, size_t workspace_bytes, void* stream) {
  if (block == nullptr || mask_strides == nullptr || counts == nullptr) return BSATTN_ERR_NULL;
  int rc = fwd_check(q, k, v, o, row_ptr, col_idx, Bm, Hm, B, H, N, D, dtype, out_dtype, q_strides, k_strides,
                     v_strides, o_strides);
  if (rc != BSATTN_OK) return rc;
  size_t need = 0;
  if ((rc = bsattn_fwd_block_mask_workspace(Bm, Hm, B, H, N, D, &need)) != BSATTN_OK) return rc;
  if (workspace == nullptr || workspace_bytes < need) return BSATTN_ERR_WORKSPACE;
  if (((uintptr_t)workspace & 15) != 0) return BSATTN_ERR_STRIDE;
  const int nb = N / BSATTN_TILE;
  rc = launch_block_mask_to_lists(block, Bm, Hm, nb, mask_strides[0], mask_strides[1], mask_strides[2], mask_strides[3],
                                  row_ptr, col_idx, nullptr, counts, (int32_t*)workspace, (hipStream_t)stream);
  if (rc != BSATTN_OK) return rc;
  AttnShape s;
  s.B = B; s.H = H; s.N = N; s.D = D; s.Bm = Bm; s.Hm = Hm; s.dtype = dtype; s.out_dtype = out_dtype;
  s.sm_scale = sm_scale;
  for (int i = 0; i < 3; ++i) { s.qs[i] = q_strides[i]; s.ks[i] = k_strides[i]; s.vs[i] = v_strides[i]; s.os[i] = o_strides[i]; s.dos[i] = 0; }
  return launch_fwd(q, k, v, o, lse, row_ptr, col_idx, nullptr, nullptr, s, (char*)workspace + lists_part_bytes(Bm, Hm, nb),
                    (hipStream_t)stream);
}

int bsattn_fwd_static(const void* q, const void* k, const void* v, void* o, float* lse,
                      const int32_t* row_ptr, const int32_t* col_idx, int Bm, int Hm, int B, int H, int N,
                      int D, int dtype, int out_dtype, float sm_scale, const int64_t* q_strides,
                      const int64_t* k_strides, const int64_t* v_strides, const int64_t* o_strides,
                      void* stream) {
  int rc = fwd_check(q, k, v, o, row_ptr, col_idx, Bm, Hm, B, H, N, D, dtype, out_dtype, q_strides, k_strides,
                     v_strides, o_strides);
  if (rc != BSATTN_OK) return rc;
  const size_t need = coop_workspace_bytes(B, H, N, D);
  if (need > (size_t)BSATTN_STATIC_SCRATCH_BYTES) return BSATTN_ERR_STATIC_LIMIT;
  void* ws = nullptr;
  if ((rc = static_scratch(&ws)) != BSATTN_OK) return rc;
  AttnShape s;
  s.B = B; s.H = H; s.N = N; s.D = D; s.Bm = Bm; s.Hm = Hm; s.dtype = dtype; s.out_dtype = out_dtype;
  s.sm_scale = sm_scale;
  for (int i = 0; i < 3; ++i) { s.qs[i] = q_strides[i]; s.ks[i] = k_strides[i]; s.vs[i] = v_strides[i]; s.os[i] = o_strides[i]; s.dos[i] = 0; }
  return launch_fwd(q, k, v, o, lse, row_ptr, col_idx, nullptr, nullptr, s, ws, (hipStream_t)stream);
}

int bsattn_fwd_elementwise(const void* q, const void* k, const void* v, void* o, float* lse,
                           const int32_t* row_ptr, const int32_t* col_idx, const uint8_t* tile_partial,
                           const uint64_t* tile_bits, int Bm, int Hm, int B, int H, int N,
                           int D, int dtype, int out_dtype, float sm_scale, const int64_t* q_strides,
                           const int64_t* k_strides, const int64_t* v_strides, const int64_t* o_strides,
                           void* workspace, size_t workspace_bytes, void* stream) {
  if (tile_partial == nullptr || tile_bits == nullptr) return BSATTN_ERR_NULL;
  if (((uintptr_t)tile_bits & 7) != 0) return BSATTN_ERR_STRIDE;
  return fwd_common(q, k, v, o, lse, row_ptr, col_idx, tile_partial, tile_bits, Bm, Hm, B, H, N, D, dtype,
                    out_dtype, sm_scale, q_strides, k_strides, v_strides, o_strides, workspace, workspace_bytes,
                    stream);
}

int bsattn_bwd_workspace(int B, int H, int N, int D, size_t* bytes) {
  if (bytes == nullptr) return BSATTN_ERR_NULL;
  const int rc = check_attn(1, 1, B, H, N, D, BSATTN_F16, BSATTN_F16);
  if (rc != BSATTN_OK) return rc;
  *bytes = bwd_workspace_bytes(B, H, N, D);
  return BSATTN_OK;
}

static int bwd_common(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                      const float* lse, void* dq, void* dk, void* dv, const int32_t* row_ptr,
                      const int32_t* col_idx, const int32_t* col_ptr, const int32_t* row_idx,
                      const uint64_t* bits_rows, const uint64_t* bits_cols, int Bm, int Hm,
                      int B, int H, int N, int D, int dtype, int out_dtype, float sm_scale,
                      const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                      const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                      const int64_t* dk_strides, const int64_t* dv_strides, void* workspace,
                      size_t workspace_bytes, void* stream) {
  if (q == nullptr || k == nullptr || v == nullptr || o == nullptr || d_o == nullptr || lse == nullptr ||
      dq == nullptr || dk == nullptr || dv == nullptr || row_ptr == nullptr || col_idx == nullptr ||
      col_ptr == nullptr || row_idx == nullptr)
    return BSATTN_ERR_NULL;
  int rc = check_attn(Bm, Hm, B, H, N, D, dtype, out_dtype);
  if (rc != BSATTN_OK) return rc;
  if ((rc = check_strides(q_strides, 2, q)) != BSATTN_OK) return rc;
  if ((rc = check_strides(k_strides, 2, k)) != BSATTN_OK) return rc;
  if ((rc = check_strides(v_strides, 2, v)) != BSATTN_OK) return rc;
  if ((rc = check_strides(o_strides, 2, o)) != BSATTN_OK) return rc;
  if ((rc = check_strides(do_strides, 2, d_o)) != BSATTN_OK) return rc;
  // results: NULL strides mean [B, H, N, D] without gaps
  const int64_t dense[4] = {(int64_t)H * N * D, (int64_t)N * D, D, 1};
  const int out_bytes = out_dtype == BSATTN_F32 ? 4 : 2;
  if (dq_strides == nullptr) dq_strides = dense;
  if (dk_strides == nullptr) dk_strides = dense;
  if (dv_strides == nullptr) dv_strides = dense;
  if ((rc = check_strides(dq_strides, out_bytes, dq)) != BSATTN_OK) return rc;
  if ((rc = check_strides(dk_strides, out_bytes, dk)) != BSATTN_OK) return rc;
  if ((rc = check_strides(dv_strides, out_bytes, dv)) != BSATTN_OK) return rc;
  if (workspace == nullptr || workspace_bytes < bwd_workspace_bytes(B, H, N, D)) return BSATTN_ERR_WORKSPACE;
  if (((uintptr_t)workspace & 15) != 0) return BSATTN_ERR_STRIDE;
  AttnShape s;
  s.B = B; s.H = H; s.N = N; s.D = D; s.Bm = Bm; s.Hm = Hm; s.dtype = dtype; s.out_dtype = out_dtype;
  s.sm_scale = sm_scale;
  for (int i = 0; i < 3; ++i) { s.qs[i] = q_strides[i]; s.ks[i] = k_strides[i]; s.vs[i] = v_strides[i]; s.os[i] = o_strides[i]; s.dos[i] = do_strides[i];
                               s.dqs[i] = dq_strides[i]; s.dks[i] = dk_strides[i]; s.dvs[i] = dv_strides[i]; }
  return launch_bwd(q, k, v, o, d_o, lse, dq, dk, dv, row_ptr, col_idx, col_ptr, row_idx, bits_rows, bits_cols, s,
                    workspace, (hipStream_t)stream);
}

int bsattn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
               const float* lse, void* dq, void* dk, void* dv, const int32_t* row_ptr,
               const int32_t* col_idx, const int32_t* col_ptr, const int32_t* row_idx, int Bm, int Hm,
               int B, int H, int N, int D, int dtype, int out_dtype, float sm_scale,
               const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
               const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
               const int64_t* dk_strides, const int64_t* dv_strides, void* workspace,
               size_t workspace_bytes, void* stream) {
  return bwd_common(q, k, v, o, d_o, lse, dq, dk, dv, row_ptr, col_idx, col_ptr, row_idx, nullptr, nullptr, Bm, Hm,
                    B, H, N, D, dtype, out_dtype, sm_scale, q_strides, k_strides, v_strides, o_strides, do_strides,
                    dq_strides, dk_strides, dv_strides, workspace, workspace_bytes, stream);
}

int bsattn_bwd_elementwise(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                           const float* lse, void* dq, void* dk, void* dv, const int32_t* row_ptr,
                           const int32_t* col_idx, const int32_t* col_ptr, const int32_t* row_idx,
                           const uint64_t* tile_bits_rows, const uint64_t* tile_bits_cols, int Bm, int Hm,
                           int B, int H, int N, int D, int dtype, int out_dtype, float sm_scale,
                           const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                           const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                           const int64_t* dk_strides, const int64_t* dv_strides, void* workspace,
                           size_t workspace_bytes, void* stream) {
  if (tile_bits_rows == nullptr || tile_bits_cols == nullptr) return BSATTN_ERR_NULL;
  if ((((uintptr_t)tile_bits_rows | (uintptr_t)tile_bits_cols) & 7) != 0) return BSATTN_ERR_STRIDE;
  return bwd_common(q, k, v, o, d_o, lse, dq, dk, dv, row_ptr, col_idx, col_ptr, row_idx, tile_bits_rows,
                    tile_bits_cols, Bm, Hm, B, H, N, D, dtype, out_dtype, sm_scale, q_strides, k_strides, v_strides,
                    o_strides, do_strides, dq_strides, dk_strides, dv_strides, workspace, workspace_bytes, stream);
}

int bsattn_reorder(const void* x, void* out, int BS, int NH, int F, int Hh, int W, int D, int elem_bytes,
                   const int32_t* orders, const int32_t* inv_orders, void* stream) {
  if (x == nullptr || out == nullptr || orders == nullptr) return BSATTN_ERR_NULL;
  if (BS <= 0 || NH <= 0 || F <= 0 || Hh <= 0 || W <= 0 || D <= 0 || elem_bytes <= 0) return BSATTN_ERR_SHAPE;
  const int64_t row_bytes = (int64_t)D * elem_bytes;
  if (row_bytes % 4 != 0 || ((uintptr_t)x & 3) != 0 || ((uintptr_t)out & 3) != 0) return BSATTN_ERR_STRIDE;
  if ((int64_t)BS * NH * F * Hh * W > 0x7fffffffLL || row_bytes > 0x7fffffffLL) return BSATTN_ERR_RANGE;
  return launch_reorder(x, out, BS, NH, F, Hh, W, (int)row_bytes, orders, inv_orders, (hipStream_t)stream);
}

}  // extern "C"
