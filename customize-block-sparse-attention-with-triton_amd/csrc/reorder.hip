// Head-wise token reorder: out[b,h,new_t,:] = x[b,h,t,:], a pure HBM-bound row gather.
// Index arithmetic follows fa2_custom_mask/permute.py:20-52 (forward) and :77-120 (inverse);
// unlike the reference's scalar loop over the head dimension (:54-58) a token row is moved
// with coalesced vector accesses: consecutive lanes copy consecutive 16-byte (or 4-byte)
// pieces of one row.
#include "common.h"

namespace bsattn {

__device__ __forceinline__ int64_t new_token(int f, int h_, int w, int d0, int d1, int d2, int p0,
                                             int p1, int p2) {
  const int c0 = p0 == 0 ? f : (p0 == 1 ? h_ : w);
  const int c1 = p1 == 0 ? f : (p1 == 1 ? h_ : w);
  const int c2 = p2 == 0 ? f : (p2 == 1 ? h_ : w);
  const int e1 = p1 == 0 ? d0 : (p1 == 1 ? d1 : d2);
  const int e2 = p2 == 0 ? d0 : (p2 == 1 ? d1 : d2);
  return (int64_t)c0 * (e1 * e2) + (int64_t)c1 * e2 + c2;  // permute.py:45-52
}

template <typename V>
__global__ __launch_bounds__(256) void reorder_kernel(const V* __restrict__ x, V* __restrict__ out,
                                                      int64_t total_rows, int NH, int F, int Hh, int W,
                                                      int vec_per_row, const int32_t* __restrict__ orders,
                                                      const int32_t* __restrict__ inv_orders) {
  const int T = F * Hh * W;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = gid / vec_per_row;
  const int piece = (int)(gid % vec_per_row);
  if (row >= total_rows) return;
  const int t = (int)(row % T);
  const int hd = (int)((row / T) % NH);
  int d0 = F, d1 = Hh, d2 = W;
  const int32_t* p = orders + hd * 3;
  if (inv_orders != nullptr) {  // decode t in the permuted dims (permute.py:77-95)
    const int fp = p[0], hp = p[1], wp = p[2];
    d0 = fp == 0 ? F : (fp == 1 ? Hh : W);
    d1 = hp == 0 ? F : (hp == 1 ? Hh : W);
    d2 = wp == 0 ? F : (wp == 1 ? Hh : W);
    p = inv_orders + hd * 3;
  }
  const int f = t / (d1 * d2), t_ = t % (d1 * d2), h_ = t_ / d2, w = t_ % d2;
  const int64_t nt = new_token(f, h_, w, d0, d1, d2, p[0], p[1], p[2]);
  const int64_t orow = row - t + nt;
  out[orow * vec_per_row + piece] = x[row * vec_per_row + piece];
}

int launch_reorder(const void* x, void* out, int BS, int NH, int F, int Hh, int W, int row_bytes,
                   const int32_t* orders, const int32_t* inv_orders, hipStream_t st) {
  const int64_t rows = (int64_t)BS * NH * F * Hh * W;
  typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));
  const bool v16 = row_bytes % 16 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0;
  const int vpr = v16 ? row_bytes / 16 : row_bytes / 4;
  const int64_t threads = rows * vpr;
  const dim3 grid((unsigned)((threads + 255) / 256));
  if (v16)
    hipLaunchKernelGGL(reorder_kernel<uintx4>, grid, dim3(256), 0, st, (const uintx4*)x, (uintx4*)out, rows,
                       NH, F, Hh, W, vpr, orders, inv_orders);
  else
    hipLaunchKernelGGL(reorder_kernel<unsigned int>, grid, dim3(256), 0, st, (const unsigned int*)x,
                       (unsigned int*)out, rows, NH, F, Hh, W, vpr, orders, inv_orders);
  return launch_status();
}

}  // namespace bsattn
