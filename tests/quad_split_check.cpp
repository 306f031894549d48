// Host-side check of the work split of the quad forward kernel (csrc/fwd_quad_split.h): for random
// weight axes and range counts, the ranges tile the axis, every quad's parts are the ranges
// quad_parts() names.
#include <cstdio>
#include <cstdlib>
#include <vector>
#define BSATTN_HD inline
#include "fwd_quad_split.h"
using namespace bsattn;

static unsigned long long rng_state = 88172645463325252ull;
static unsigned rnd() { rng_state ^= rng_state << 13; rng_state ^= rng_state >> 7; rng_state ^= rng_state << 17; return (unsigned)(rng_state >> 11); }

int main() {
  int cases = 0;
  for (int iter = 0; iter < 4000; ++iter) {
    const int nq = 1 + rnd() % 80, reps = 1 + rnd() % 3, maxw = 1 + rnd() % 300;
    std::vector<int32_t> cum(nq + 1, 0);
    for (int i = 0; i < nq; ++i) cum[i + 1] = cum[i] + ((rnd() % 5 == 0) ? 0 : (int)(rnd() % maxw));
    if (cum[nq] == 0) continue;
    QuadAxis ax{cum.data(), nq, cum[nq], reps, 1};
    ax.slots = quad_slots(ax.total(), 1 + rnd() % 600);
    std::vector<int64_t> cut(ax.slots + 1);
    for (int s = 0; s <= ax.slots; ++s) cut[s] = quad_cut(ax, s);
    if (cut[0] != 0 || cut[ax.slots] != ax.total()) { printf("ends\n"); return 1; }
    for (int s = 0; s < ax.slots; ++s) if (cut[s] > cut[s + 1]) { printf("order\n"); return 1; }
    // walk every range the way the kernel does and record, per quad, which ranges produced a segment
    std::vector<std::vector<int>> touched((size_t)nq * reps);
    for (int s = 0; s < ax.slots; ++s) {
      int64_t x = cut[s];
      while (x < cut[s + 1]) {
        const QuadPos p = quad_locate(ax, x);
        if (p.w <= 0 || x < p.c0 || x >= p.c0 + p.w) { printf("locate\n"); return 1; }
        const int64_t e = cut[s + 1] < p.c0 + p.w ? cut[s + 1] : p.c0 + p.w;
        touched[p.gq].push_back(s);
        x = e;
      }
    }
    for (int rep = 0; rep < reps; ++rep)
      for (int i = 0; i < nq; ++i) {
        const int w = cum[i + 1] - cum[i];
        const std::vector<int>& t = touched[(size_t)rep * nq + i];
        if (w == 0) { if (!t.empty()) { printf("empty quad touched\n"); return 1; } continue; }
        const QuadParts qp = quad_parts(ax, (int64_t)rep * cum[nq] + cum[i], w);
        if ((int)t.size() != qp.count) { printf("count %d vs %d\n", (int)t.size(), qp.count); return 1; }
        if (qp.count > 1)
          for (int k = 0; k < qp.count; ++k) if (t[k] != qp.first + k) { printf("first\n"); return 1; }
        // which of a part's range segments it is: part 0 is a later segment unless its range starts with the quad
        if (qp.count > 1 && (cut[qp.first] == (int64_t)rep * cum[nq] + cum[i]) != (cut[qp.first] >= (int64_t)rep * cum[nq] + cum[i])) { printf("which\n"); return 1; }
        ++cases;
      }
  }
  printf("ok %d quads\n", cases);
  return 0;
}
