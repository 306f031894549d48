// Partition of one head's kept-tile list into contiguous ranges, one per workgroup.
#pragma once
#include <stdint.h>

namespace bsattn {

// Where two workgroups share a compute unit, the one that arrived first gets the larger share of
// the issue slots (measured: while both run it processes tiles about 1.5 times as fast as the
// second).  The first `fast` ranges of a head therefore receive tiles in the proportion
// WEIGHT_FAST : WEIGHT_SLOW to the others.  (With 3 : 2 the first-comers finish their tiles 3 us before their
// mates on a dense head of N = 17536; 14 : 9 against it: one head 101.1 -> 100.0 us, 8 heads 696 -> 692 us;
// 20 : 13, 17 : 11 and 25 : 16 the same within 0.3 us, 11 : 7 and 8 : 5 no better than 3 : 2.)
constexpr int WEIGHT_FAST = 14, WEIGHT_SLOW = 9;
// Heads with fewer tiles per range than this are cut into equal shares.
constexpr int EQUAL_SPLIT_BELOW = 48;

struct HeadSplit {
  int lo;     // first tile of the head in the global list
  int T;      // kept tiles of the head
  int Peff;   // ranges actually used (<= P)
  int fast;   // leading ranges with the larger weight (<= Peff)
  int gap;    // what a row block boundary inside a range costs, in tiles (see below)
  int64_t ctot;  // sum of the weights
  int64_t X;     // length of the head's list on the axis the ranges are cut on: T + gap * nb
};

__device__ __forceinline__ int64_t split_cum(const HeadSplit& s, int p) {
  return p <= s.fast ? (int64_t)WEIGHT_FAST * p : (int64_t)WEIGHT_FAST * s.fast + (int64_t)WEIGHT_SLOW * (p - s.fast);
}

// The ranges are cut on an axis on which every row block is followed by `gap` positions that hold no tile: tile
// j of row block r (absolute offset rp[r] + j) sits at position rp[r] - lo + gap * r + j.  A range that goes on
// into the next row block pays for it (a merge of its wavefronts' results, a published part: several tiles'
// worth) with `gap` tiles less, and a boundary that falls into the positions behind a row block lies at the row
// block's end.  gap = 0 is the plain tile axis.
// rp: row pointers of the head (nb + 1 entries, absolute offsets)
template <typename Ptr>
__device__ __forceinline__ HeadSplit head_split(Ptr rp, int nb, int P, int min_tiles, int fast, int gap) {
  HeadSplit s;
  s.lo = rp[0];
  s.T = rp[nb] - s.lo;
  const int want = (s.T + min_tiles - 1) / min_tiles;   // no range shorter than about min_tiles
  s.Peff = want < P ? want : P;
  s.fast = fast < 0 ? 0 : (fast < s.Peff ? fast : s.Peff);
  // short ranges are a matter of latency, which both workgroups of a compute unit see alike: equal shares
  if ((int64_t)s.T < (int64_t)EQUAL_SPLIT_BELOW * s.Peff) s.fast = 0;
  s.ctot = split_cum(s, s.Peff);
  s.gap = gap;
  s.X = (int64_t)s.T + (int64_t)gap * nb;
  return s;
}

// position on the cutting axis where range p begins (p == Peff gives X); requires T > 0
__device__ __forceinline__ int64_t split_pos(const HeadSplit& s, int p) {
  return (split_cum(s, p) * s.X) / s.ctot;
}

// range that contains position x, 0 <= x < X; requires T > 0
__device__ __forceinline__ int split_of_pos(const HeadSplit& s, int64_t x) {
  // y: the largest cumulative weight c with floor(X * c / ctot) <= x
  const int64_t y = ((x + 1) * s.ctot - 1) / s.X;
  const int64_t cf = (int64_t)WEIGHT_FAST * s.fast;
  return y < cf ? (int)(y / WEIGHT_FAST) : s.fast + (int)((y - cf) / WEIGHT_SLOW);
}

// position of the first tile of row block r, whose tiles are [row_s, row_e) (absolute offsets)
__device__ __forceinline__ int64_t row_pos(const HeadSplit& s, int r, int row_s) {
  return (int64_t)(row_s - s.lo) + (int64_t)s.gap * r;
}

// The tile (absolute offset) at which position x lies as seen from row block r: row_s for positions before the
// row block, row_e for positions behind its tiles.
__device__ __forceinline__ int tile_of_pos(const HeadSplit& s, int64_t x, int r, int row_s, int row_e) {
  const int64_t off = x - row_pos(s, r, row_s);
  if (off <= 0) return row_s;
  return off < (int64_t)(row_e - row_s) ? row_s + (int)off : row_e;
}

// floats per partial slot: unnormalised accumulator [64 x D] + running max [64] + sum [64]
__host__ __device__ constexpr int partial_floats(int D) { return 64 * D + 128; }

// Where a range boundary g inside the row block [s, e) of the tile list (s <= g < e) really goes: to
// the nearer end of the row block if that is at most X tiles away, else it stays.
__device__ __forceinline__ int snap_boundary(int X, int g, int s, int e) {
  const int db = g - s, df = e - g;
  if (db <= df) return db <= X ? s : g;
  return df <= X ? e : g;
}

}  // namespace bsattn
