// Shared declarations of the library's translation units (not part of the public ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include "bsattn.h"

#define BSATTN_VERSION BSATTN_ABI_VERSION

namespace bsattn {

// mask_index.hip
int launch_reduce_dense_mask(const uint8_t* dense, int Bm, int Hm, int N, int64_t sb, int64_t sh,
                             int64_t sm, uint8_t* block_out, hipStream_t st);
int launch_block_mask_to_lists(const uint8_t* block, int Bm, int Hm, int nb, int64_t sb, int64_t sh,
                               int64_t sm, int64_t sn, int32_t* row_ptr, int32_t* col_idx,
                               int32_t* groups, int32_t* counts, int32_t* ws, hipStream_t st);

int launch_tail_tiles(int Bm, int Hm, int nb, int valid, int transpose, const int32_t* row_ptr,
                      const int32_t* col_idx, uint8_t* partial, unsigned long long* bits, hipStream_t st);
int launch_reduce_pack(const uint8_t* dense, int Bm, int Hm, int N, int64_t sb, int64_t sh, int64_t sm,
                       uint8_t* block_out, uint8_t* grid_partial, unsigned long long* grid_bits, hipStream_t st);
int launch_gather_tiles(const uint8_t* grid_partial, const unsigned long long* grid_bits, int Bm, int Hm, int nb,
                        int transposed, const int32_t* row_ptr, const int32_t* col_idx, uint8_t* partial,
                        unsigned long long* bits, hipStream_t st);
int launch_pack_tiles(const uint8_t* dense, int Bm, int Hm, int nb, int64_t sb, int64_t sh, int64_t sm,
                      int64_t sn, const int32_t* row_ptr, const int32_t* col_idx, uint8_t* partial,
                      unsigned long long* bits, hipStream_t st);

struct AttnShape {
  int B, H, N, D, Bm, Hm;
  int dtype, out_dtype;
  float sm_scale;
  int64_t qs[3], ks[3], vs[3], os[3], dos[3];  // batch, head, row strides (elements)
  int64_t dqs[3], dks[3], dvs[3];              // ... of the backward's results
};

// attn_fwd.hip
int compute_units();   // of the current device (256 if the query fails)

// Runs f unless it has completed before for the current device (one `done` mask per call site):
// kernel attributes such as the dynamic LDS limit are kept per device.  Two threads may both run
// f for a device; f must be idempotent.
template <class F>
inline void once_per_device(std::atomic<unsigned long long>& done, F&& f) {
  int dev = 0;
  (void)hipGetDevice(&dev);
  const unsigned long long bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return;
  f();
  done.fetch_or(bit, std::memory_order_release);
}
size_t fwd_workspace_bytes(int B, int H, int N, int D);
unsigned long long next_epoch();   // a 48-bit number that differs from launch to launch, never zero
int set_deterministic(int on);   // returns the previous setting
int get_deterministic();
int launch_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
               const int32_t* row_ptr, const int32_t* col_idx, const uint8_t* tile_partial,
               const uint64_t* tile_bits, const AttnShape& s, void* ws, hipStream_t st);
size_t coop_workspace_bytes(int B, int H, int N, int D);   // what launch_fwd itself needs
// Address, on the current device, of the library's own scratch array (BSATTN_STATIC_SCRATCH_BYTES).
int static_scratch(void** ptr);

// attn_bwd.hip
size_t bwd_workspace_bytes(int B, int H, int N, int D);
int launch_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
               const float* lse, void* dq, void* dk, void* dv, const int32_t* row_ptr,
               const int32_t* col_idx, const int32_t* col_ptr, const int32_t* row_idx,
               const uint64_t* bits_rows, const uint64_t* bits_cols,
               const AttnShape& s, void* ws, hipStream_t st);

// reorder.hip
int launch_reorder(const void* x, void* out, int BS, int NH, int F, int Hh, int W, int row_bytes,
                   const int32_t* orders, const int32_t* inv_orders, hipStream_t st);

inline int launch_status() { return hipGetLastError() == hipSuccess ? BSATTN_OK : BSATTN_ERR_LAUNCH; }

}  // namespace bsattn
