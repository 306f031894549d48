// Partition of one head's kept-tile list into contiguous ranges, one per workgroup.
#pragma once
#include <stdint.h>

namespace bsattn {

// Where two workgroups share a compute unit, the one that arrived first gets the larger share of
// the issue slots (measured: while both run it processes tiles about 1.5 times as fast as the
// second).  The first `fast` ranges of a head therefore receive tiles in the proportion
// WEIGHT_FAST : WEIGHT_SLOW to the others.
constexpr int WEIGHT_FAST = 3, WEIGHT_SLOW = 2;

struct HeadSplit {
  int lo;     // first tile of the head in the global list
  int T;      // kept tiles of the head
  int Peff;   // ranges actually used (<= P)
  int fast;   // leading ranges with the larger weight (<= Peff)
  int64_t ctot;  // sum of the weights
};

__device__ __forceinline__ int64_t split_cum(const HeadSplit& s, int p) {
  return p <= s.fast ? (int64_t)WEIGHT_FAST * p : (int64_t)WEIGHT_FAST * s.fast + (int64_t)WEIGHT_SLOW * (p - s.fast);
}

// rp: row pointers of the head (nb + 1 entries, absolute offsets)
template <typename Ptr>
__device__ __forceinline__ HeadSplit head_split(Ptr rp, int nb, int P, int min_tiles, int fast) {
  HeadSplit s;
  s.lo = rp[0];
  s.T = rp[nb] - s.lo;
  const int want = (s.T + min_tiles - 1) / min_tiles;   // no range shorter than about min_tiles
  s.Peff = want < P ? want : P;
  s.fast = fast < 0 ? 0 : (fast < s.Peff ? fast : s.Peff);
#ifndef EQUAL_SPLIT_BELOW
#define EQUAL_SPLIT_BELOW 48
#endif
  // short ranges are a matter of latency, which both workgroups of a compute unit see alike: equal shares
  if ((int64_t)s.T < (int64_t)EQUAL_SPLIT_BELOW * s.Peff) s.fast = 0;
  s.ctot = split_cum(s, s.Peff);
  return s;
}

// first tile of range p (p == Peff gives the end of the list); requires T > 0
__device__ __forceinline__ int split_begin(const HeadSplit& s, int p) {
  return s.lo + (int)((split_cum(s, p) * s.T) / s.ctot);
}

// range that contains tile t (absolute offset); requires T > 0
__device__ __forceinline__ int split_of_tile(const HeadSplit& s, int t) {
  // y: the largest cumulative weight c with floor(T * c / ctot) <= t - lo
  const int64_t y = (((int64_t)(t - s.lo) + 1) * s.ctot - 1) / s.T;
  const int64_t cf = (int64_t)WEIGHT_FAST * s.fast;
  return y < cf ? (int)(y / WEIGHT_FAST) : s.fast + (int)((y - cf) / WEIGHT_SLOW);
}

// floats per partial slot: unnormalised accumulator [64 x D] + running max [64] + sum [64]
__host__ __device__ constexpr int partial_floats(int D) { return 64 * D + 128; }

// Where a range boundary g inside the row block [s, e) of the tile list (s <= g < e) really goes: to
// the nearer end of the row block if that is at most X tiles away, else it stays.
template <int X>
__device__ __forceinline__ int snap_boundary(int g, int s, int e) {
  const int db = g - s, df = e - g;
  if (db <= df) return db <= X ? s : g;
  return df <= X ? e : g;
}

}  // namespace bsattn
