// Host-side check of the range permutation of the forward kernel (csrc/range_perm.h): for many list shapes the
// table is a bijection of the ranges that keeps the two weight classes apart, and the ranges it gives to the
// workgroups of one XCD form one run of the class's ranges sorted by phase.
#include <cstdio>
#include <cstdint>
#include <vector>
#include "range_perm.h"
using namespace bsattn;

int main() {
  int made = 0, refused = 0;
  const int wf = 3, ws = 2;
  for (int BH : {1, 2, 3, 4, 8})
    for (int W = 1; W <= 520; W += (W < 40 ? 1 : 7))
      for (int F : {0, W / 4, W / 2, W})
        for (int nb : {1, 2, 16, 100, 137, 274, 500, 2048}) {
         for (int causal = 0; causal < 2; ++causal) {
          std::vector<unsigned short> t(RANGE_PERM_MAX + 8, 0xffff);
          const bool ok = make_range_permutation(nb, W, F, BH, wf, ws, causal != 0, t.data());
          for (int i = (ok ? W : 0); i < (int)t.size(); ++i) if (t[i] != 0xffff) { printf("wrote past the table\n"); return 1; }
          if (!ok) { ++refused; continue; }
          ++made;
          const int nx = 8 / BH;
          std::vector<int> seen(W, 0);
          for (int wg = 0; wg < W; ++wg) {
            const int p = t[wg];
            if (p >= W || seen[p]++) { printf("not a bijection: nb %d W %d F %d BH %d\n", nb, W, F, BH); return 1; }
            if ((wg < F) != (p < F)) { printf("classes mixed: nb %d W %d F %d BH %d\n", nb, W, F, BH); return 1; }
          }
          auto cum = [&](int p) { return p <= F ? (int64_t)wf * p : (int64_t)wf * F + (int64_t)ws * (p - F); };
          const int64_t ctot = cum(W);
          auto phase = [&](int p) {
            if (!causal) return (cum(p) * nb) % ctot;
            const int64_t T = (int64_t)nb * (nb + 1) / 2, tile = cum(p) * T / ctot;
            int64_t r = 0;
            while ((r + 1) * (r + 2) / 2 <= tile) ++r;       // (brute force: the row the tile lies in)
            return tile - r * (r + 1) / 2;
          };
          for (int cls = 0; cls < 2; ++cls) {
            const int base = cls == 0 ? 0 : F, n = cls == 0 ? F : W - F;
            // largest phase on XCD x must not exceed the smallest phase on XCD x + 1
            std::vector<int64_t> lo(nx, INT64_MAX), hi(nx, -1);
            std::vector<int> cnt(nx, 0);
            for (int i = 0; i < n; ++i) {
              const int x = (base + i) % nx;
              const int64_t ph = phase(t[base + i]);
              if (ph < lo[x]) lo[x] = ph;
              if (ph > hi[x]) hi[x] = ph;
              ++cnt[x];
            }
            for (int x = 0; x < nx; ++x) {
              if (n > 0 && cnt[x] != n / nx) { printf("uneven: nb %d W %d F %d BH %d\n", nb, W, F, BH); return 1; }
              if (n > 0 && x + 1 < nx && hi[x] > lo[x + 1]) { printf("runs overlap: nb %d W %d F %d BH %d\n", nb, W, F, BH); return 1; }
            }
          }
         }
        }
  if (made < 200 || refused < 200) { printf("too few cases: %d made, %d refused\n", made, refused); return 1; }
  printf("range permutation: %d tables checked, %d shapes refused\nok\n", made, refused);
  return 0;
}
