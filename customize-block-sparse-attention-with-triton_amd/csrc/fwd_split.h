// Partition of one head's kept-tile list into equal contiguous ranges, shared by the kernels
// that produce partial results and the kernels that merge them.
#pragma once
#include <stdint.h>

namespace bsattn {


struct HeadSplit {
  int lo;    // first tile of the head in the global list
  int T;     // kept tiles of the head
  int Peff;  // ranges actually used (<= P)
};

// rp: row pointers of the head (nb + 1 entries, absolute offsets)
template <typename Ptr>
__device__ __forceinline__ HeadSplit head_split(Ptr rp, int nb, int P, int min_tiles) {
  HeadSplit s;
  s.lo = rp[0];
  s.T = rp[nb] - s.lo;
  const int want = (s.T + min_tiles - 1) / min_tiles;   // no range shorter than min_tiles
  s.Peff = want < P ? want : P;
  return s;
}

// first tile of range p (p == Peff gives the end of the list)
__device__ __forceinline__ int split_begin(const HeadSplit& s, int p) {
  return s.lo + (int)(((int64_t)p * s.T) / s.Peff);
}

// range that contains tile t (absolute offset); requires T > 0
__device__ __forceinline__ int split_of_tile(const HeadSplit& s, int t) {
  return (int)((((int64_t)(t - s.lo) + 1) * s.Peff - 1) / s.T);
}

// floats per partial slot: unnormalised accumulator [64 x D] + running max [64] + sum [64]
__host__ __device__ constexpr int partial_floats(int D) { return 64 * D + 128; }

}  // namespace bsattn
