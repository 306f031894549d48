// Which range of a head's tile list each workgroup of fwd_kernel takes (host side, plain C++).
//
// A head's list is cut into W ranges, the first F of weight wf, the others of weight ws (fwd_split.h); range p
// starts at the fraction cum(p) / cum(W) of the list, cum(p) = wf * min(p, F) + ws * max(p - F, 0), which for
// rows of equal length is the phase frac(cum(p) * nb / cum(W)) of a row.  Workgroups go to the 8 XCDs of the GPU
// round-robin by linear id (wg * BH + bh for BH heads), so workgroup wg of a head sits on the head's XCD number
// wg % nx, nx = 8 / BH.  Within each weight class (the first-come, faster workgroups keep the larger ranges) the
// ranges are sorted by phase and dealt out in nx equal runs, one per XCD: the workgroups that share an L2 then
// walk the same column blocks at the same time.
#pragma once
#include <algorithm>
#include <cstdint>
#include <utility>
#include <vector>

namespace bsattn {

constexpr int RANGE_PERM_MAX = 512;

// For the other mask that is all long rows, the dense block-causal one (row r keeps columns 0 .. r), the ranges
// are sorted by the column block they start at instead: range p starts at tile floor(cum(p) T / cum(W)) of the
// T = nb (nb + 1) / 2 kept tiles (the kernel's split_begin), which lies in the row r with r (r + 1) / 2 <= tile.
//
// out[wg] = range of workgroup wg, for wg < W.  False (out untouched) where no such table applies: more than 4
// or not 1, 2, 4 heads, more than RANGE_PERM_MAX ranges, classes that do not split evenly over the XCDs.
inline bool make_range_permutation(int nb, int W, int F, int BH, int wf, int ws, bool block_causal, unsigned short* out) {
  if (BH != 1 && BH != 2 && BH != 4) return false;
  const int nx = 8 / BH;
  if (nb <= 0 || W > RANGE_PERM_MAX || W < 2 * nx || F < 0 || F > W || F % nx != 0 || (W - F) % nx != 0) return false;
  auto cum = [&](int p) { return p <= F ? (int64_t)wf * p : (int64_t)wf * F + (int64_t)ws * (p - F); };
  const int64_t ctot = cum(W);
  if (ctot <= 0) return false;
  for (int cls = 0; cls < 2; ++cls) {
    const int base = cls == 0 ? 0 : F, n = cls == 0 ? F : W - F;
    if (n == 0) continue;
    std::vector<std::pair<int64_t, int>> order(n);
    for (int i = 0; i < n; ++i) {
      int64_t key = (cum(base + i) * nb) % ctot;
      if (block_causal) {
        const int64_t T = (int64_t)nb * (nb + 1) / 2, tile = cum(base + i) * T / ctot;
        int64_t r = 0;
        for (int64_t step = (int64_t)1 << 20; step > 0; step >>= 1)       // largest r with r (r + 1) / 2 <= tile
          if ((r + step) * (r + step + 1) / 2 <= tile) r += step;
        key = tile - r * (r + 1) / 2;
      }
      order[i] = {key, base + i};
    }
    std::sort(order.begin(), order.end());
    // workgroup base + i: XCD (base + i) % nx = i % nx (base is a multiple of nx), the (i / nx)-th of its class there
    for (int i = 0; i < n; ++i) out[base + i] = (unsigned short)order[(size_t)(i % nx) * (n / nx) + i / nx].second;
  }
  return true;
}

}  // namespace bsattn
