// Drives the argument validation of the C ABI (include/bsattn.h) in a build whose host code carries the
// address and undefined-behaviour sanitizers: every call below must be refused before any device work, so
// the program needs no GPU.  Pointers that are never dereferenced point at a small real buffer, so that a
// validation path that did read them would be caught.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include "bsattn.h"

static int failures = 0;
#define EXPECT(call, want) do { const int rc_ = (call); if (rc_ != (want)) { \
  std::printf("line %d: %s returned %d, expected %d\n", __LINE__, #call, rc_, (int)(want)); ++failures; } } while (0)

int main() {
  alignas(16) static unsigned char buf[64];
  void* P = buf;
  const int64_t ok[4] = {64 * 64, 64 * 64, 64, 1}, inner2[4] = {64 * 64, 64 * 64, 64, 2}, odd[4] = {64 * 68, 64 * 68, 68, 1};
  size_t n = 0;
  const size_t big = (size_t)1 << 40;
  auto fwd = [&](const void* q, const void* rp, int Bm, int B, int N, int D, int dt, int odt, const int64_t* qs,
                 const int64_t* ks, void* ws, size_t wsb) {
    return bsattn_fwd(q, P, P, P, nullptr, (const int32_t*)rp, (const int32_t*)P, Bm, 1, B, 1, N, D, dt, odt, 0.125f, qs, ks, ok, ok,
                      ws, wsb, nullptr);
  };
  EXPECT(fwd(nullptr, P, 1, 1, 64, 64, 0, 0, ok, ok, P, big), BSATTN_ERR_NULL);
  EXPECT(fwd(P, nullptr, 1, 1, 64, 64, 0, 0, ok, ok, P, big), BSATTN_ERR_NULL);
  EXPECT(fwd(P, P, 1, 1, 100, 64, 0, 0, ok, ok, P, big), BSATTN_ERR_SHAPE);
  EXPECT(fwd(P, P, 1, 0, 64, 64, 0, 0, ok, ok, P, big), BSATTN_ERR_SHAPE);
  EXPECT(fwd(P, P, 3, 2, 64, 64, 0, 0, ok, ok, P, big), BSATTN_ERR_SHAPE);
  EXPECT(fwd(P, P, 1, 1, 64, 64, 5, 0, ok, ok, P, big), BSATTN_ERR_DTYPE);
  EXPECT(fwd(P, P, 1, 1, 64, 64, 0, 1, ok, ok, P, big), BSATTN_ERR_DTYPE);
  EXPECT(fwd(P, P, 1, 1, 64, 96, 0, 0, ok, ok, P, big), BSATTN_ERR_HEAD_DIM);
  EXPECT(fwd(P, P, 1, 1, 64, 64, 0, 0, inner2, ok, P, big), BSATTN_ERR_STRIDE);
  EXPECT(fwd(P, P, 1, 1, 64, 64, 0, 0, ok, odd, P, big), BSATTN_ERR_STRIDE);
  EXPECT(fwd(buf + 2, P, 1, 1, 64, 64, 0, 0, ok, ok, P, big), BSATTN_ERR_STRIDE);
  EXPECT(fwd(P, P, 1, 1, 64, 64, 0, 0, ok, ok, nullptr, big), BSATTN_ERR_WORKSPACE);
  EXPECT(fwd(P, P, 1, 1, 64, 64, 0, 0, ok, ok, P, 16), BSATTN_ERR_WORKSPACE);
  EXPECT(bsattn_fwd_workspace(1, 1, 100, 64, &n), BSATTN_ERR_SHAPE);
  EXPECT(bsattn_fwd_workspace(1, 1, 128, 64, nullptr), BSATTN_ERR_NULL);
  EXPECT(bsattn_fwd_workspace(1, 1, 17536, 64, &n), BSATTN_OK);
  EXPECT(bsattn_bwd_workspace(1, 1, 17536, 128, &n), BSATTN_OK);
  EXPECT(bsattn_mask_lists_workspace(1, 1, 0, &n), BSATTN_ERR_SHAPE);
  EXPECT(bsattn_mask_lists_workspace(64, 64, 4096, &n), BSATTN_ERR_RANGE);
  EXPECT(bsattn_fwd_static(P, P, P, P, nullptr, (const int32_t*)P, (const int32_t*)P, 1, 1, 1, 1, 17536, 256, 0, 0, 0.1f, ok, ok, ok,
                           ok, nullptr), BSATTN_ERR_STATIC_LIMIT);
  EXPECT(bsattn_bwd(P, P, P, P, P, (const float*)P, P, P, nullptr, (const int32_t*)P, (const int32_t*)P, (const int32_t*)P,
                    (const int32_t*)P, 1, 1, 1, 1, 64, 64, 0, 0, 0.1f, ok, ok, ok, ok, ok, nullptr, nullptr, nullptr, P, big,
                    nullptr), BSATTN_ERR_NULL);
  EXPECT(bsattn_bwd(P, P, P, P, P, (const float*)P, P, P, P, (const int32_t*)P, (const int32_t*)P, (const int32_t*)P,
                    (const int32_t*)P, 1, 1, 1, 1, 64, 64, 0, 0, 0.1f, ok, ok, ok, ok, ok, inner2, nullptr, nullptr, P, big,
                    nullptr), BSATTN_ERR_STRIDE);
  EXPECT(bsattn_bwd(P, P, P, P, P, (const float*)P, P, P, P, (const int32_t*)P, (const int32_t*)P, (const int32_t*)P,
                    (const int32_t*)P, 1, 1, 1, 1, 64, 64, 0, 0, 0.1f, ok, ok, ok, ok, ok, nullptr, nullptr, nullptr, P, 16,
                    nullptr), BSATTN_ERR_WORKSPACE);
  for (int c = -10; c <= 0; ++c)
    if (bsattn_strerror(c) == nullptr || std::strlen(bsattn_strerror(c)) == 0) { std::printf("strerror %d\n", c); ++failures; }
  EXPECT(bsattn_set_deterministic(1), 0);
  EXPECT(bsattn_set_deterministic(0), 1);
  if (failures == 0) std::printf("ok\n");
  return failures != 0;
}
