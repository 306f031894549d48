// Work split of the quad forward kernel (attn_fwd_quad.hip): plain integer arithmetic, shared by the
// kernel and by a host-side test.
//
// Four consecutive row blocks of a head form a quad; the quad's weight is the number of key tiles that
// any of its four row blocks keeps (the length of the walk over the union of their lists).  The quads of a launch, in (batch, head, quad) order, lie one after the other
// on a weight axis; `cum` holds the prefix sums over the quads of one period (all quads of the
// launch, or the quads of one head when every head uses the same mask, in which case the axis
// repeats the period `reps` times).  The axis is cut into `slots` equal ranges, one per wavefront
// group; a cut that falls within QUAD_SNAP of an end of its quad moves to that end.
#pragma once
#include <stdint.h>

#ifndef BSATTN_HD
#define BSATTN_HD __host__ __device__ __forceinline__
#endif

namespace bsattn {

constexpr int QUAD_SNAP = 3;        // cuts this close to a quad end move there
constexpr int QUAD_MIN_STEPS = 8;   // no range shorter than this (> 2 QUAD_SNAP: cuts keep their order)

struct QuadAxis {
  const int32_t* cum;   // [period_quads + 1], cum[0] = 0
  int period_quads;     // quads per period
  int period_weight;    // cum[period_quads] (> 0)
  int reps;             // periods on the axis
  int slots;            // ranges the axis is cut into (>= 1)
  BSATTN_HD int64_t total() const { return (int64_t)period_weight * reps; }
  BSATTN_HD int find(int xr) const {
    int lo = 0, hi = period_quads;            // invariant: cum[lo] <= xr < cum[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (cum[mid] <= xr) lo = mid; else hi = mid;
    }
    return lo;
  }
};

// number of ranges for an axis of `total` weight when `max_slots` wavefront groups exist
BSATTN_HD int quad_slots(int64_t total, int max_slots) {
  int64_t s = total / QUAD_MIN_STEPS;
  if (s < 1) s = 1;
  return (int)(s < max_slots ? s : max_slots);
}

struct QuadPos {
  int gq;        // global quad index (rep * period_quads + index within the period)
  int64_t c0;    // weight position where the quad starts
  int w;         // its weight (> 0)
};

// The quad with c0 <= x < c0 + w (quads of weight 0 are never returned); requires 0 <= x < total.
// ax.find(xr) returns the largest i in [0, period_quads) with cum[i] <= xr (xr < period_weight).
template <typename Axis>
BSATTN_HD QuadPos quad_locate(const Axis& ax, int64_t x) {
  const int rep = (int)(x / ax.period_weight);
  const int xr = (int)(x - (int64_t)rep * ax.period_weight);
  const int lo = ax.find(xr);
  QuadPos p;
  p.gq = rep * ax.period_quads + lo;
  p.c0 = (int64_t)rep * ax.period_weight + ax.cum[lo];
  p.w = ax.cum[lo + 1] - ax.cum[lo];
  return p;
}

// cut s of the axis (0 <= s <= slots), snapped
template <typename Axis>
BSATTN_HD int64_t quad_cut(const Axis& ax, int s) {
  const int64_t total = ax.total();
  if (s <= 0) return 0;
  if (s >= ax.slots) return total;
  const int64_t x = (total * s) / ax.slots;
  const QuadPos p = quad_locate(ax, x);
  const int64_t d0 = x - p.c0, d1 = p.c0 + p.w - x;
  if (d0 <= d1) return d0 <= QUAD_SNAP ? p.c0 : x;
  return d1 <= QUAD_SNAP ? p.c0 + p.w : x;
}

// The ranges that share the quad [c0, c0 + w): `count` ranges that follow each other, starting with
// range `first` (count == 1: the quad lies inside one range, and `first` is not set).  A cut lies
// strictly inside the quad exactly if its unsnapped position is more than QUAD_SNAP away from both
// ends (any other cut is moved to an end of this quad, or lies in another quad and stays there).
struct QuadParts { int first, count; };
template <typename Axis>
BSATTN_HD QuadParts quad_parts(const Axis& ax, int64_t c0, int w) {
  const int64_t total = ax.total(), n = ax.slots;
  const int64_t a = c0 + QUAD_SNAP, b = c0 + w - QUAD_SNAP;     // inside: a < floor(total s / n) < b
  QuadParts r;
  r.first = -1;
  r.count = 1;
  if (b - a < 2) return r;
  int64_t s_lo = ((a + 1) * n + total - 1) / total;             // smallest s with floor(total s / n) >= a + 1
  int64_t s_hi = (b * n + total - 1) / total - 1;               // largest s with total s / n < b
  if (s_lo < 1) s_lo = 1;
  if (s_hi > n - 1) s_hi = n - 1;
  if (s_lo > s_hi) return r;
  r.first = (int)s_lo - 1;
  r.count = (int)(s_hi - s_lo) + 2;
  return r;
}

}  // namespace bsattn
