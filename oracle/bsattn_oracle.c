/* CPU oracle, plain C.  TEST INFRASTRUCTURE ONLY: the shipped library never links or
 * calls this file; tests, the smoke entry and the benchmark's cpu_baseline leg do.
 *
 * Restates (paths relative to the reference repository root):
 *   oracle_build_groups   fa2_custom_mask/fa2_custom_mask.py:15-38
 *   oracle_naive_fwd      kernel-test.py:37-40 with the mask expansion of :18
 *   oracle_reorder        fa2_custom_mask/permute.py:5-58
 *   oracle_inv_reorder    fa2_custom_mask/permute.py:60-126
 * Pinned against the numpy oracle, which is itself pinned against library closed forms and
 * the hand-worked fixture: tests/test_oracle_index.py (oracle_build_groups),
 * tests/test_oracle_attention.py (oracle_naive_fwd), tests/test_oracle_reorder.py (the reorders).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define TILE 64

/* mask: bool bytes [B,H,nb,nb] contiguous.  groups: capacity B*H*nb*5, n_list: capacity
 * B*H*nb*nb.  Writes G and T; returns 0.  (G == 0 is the reference's (None, None).) */
int oracle_build_groups(const uint8_t* mask, int B, int H, int nb,
                        int32_t* groups, int32_t* n_list, int64_t* G_out, int64_t* T_out) {
  int64_t G = 0, T = 0;
  for (int b = 0; b < B; ++b)                                   /* :24 */
    for (int h = 0; h < H; ++h)                                 /* :25 */
      for (int m = 0; m < nb; ++m) {                            /* :27 */
        const uint8_t* row = mask + (((int64_t)b * H + h) * nb + m) * nb;
        int64_t start = T;                                      /* :31 */
        int len = 0;
        for (int n = 0; n < nb; ++n)                            /* :28 */
          if (row[n]) { n_list[T++] = n; ++len; }               /* :32 */
        if (len == 0) continue;                                 /* :29-30 */
        int32_t* g = groups + G * 5;                            /* :33 */
        g[0] = b; g[1] = h; g[2] = m; g[3] = (int32_t)start; g[4] = len;
        ++G;
      }
  *G_out = G; *T_out = T;
  return 0;
}

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* q,k,v,o: fp32 [BH, N, D] contiguous; mask: bool bytes [BHm, nb, nb] with BHm == BH or 1
 * (shared mask).  Processes query rows [row0,row1) of every head (a bounded sample of the
 * workload when row1-row0 < N).  lse may be NULL. */
int oracle_naive_fwd(const float* q, const float* k, const float* v, const uint8_t* mask,
                     int BH, int BHm, int N, int D, float sm_scale, int row0, int row1,
                     float* o, float* lse) {
  if (N % TILE) return -1;
  const int nb = N / TILE;
#pragma omp parallel
  {
    float* s = (float*)malloc(sizeof(float) * (size_t)N);
#pragma omp for collapse(2) schedule(dynamic, 16)
    for (int bh = 0; bh < BH; ++bh)
      for (int r = row0; r < row1; ++r) {
        const float* qr = q + ((int64_t)bh * N + r) * D;
        const float* kb = k + (int64_t)bh * N * D;
        const float* vb = v + (int64_t)bh * N * D;
        const uint8_t* mrow = mask + ((int64_t)(BHm == 1 ? 0 : bh) * nb + r / TILE) * nb;
        float mx = -INFINITY;
        for (int c = 0; c < N; ++c) {                           /* kernel-test.py:37-38 */
          float acc = -INFINITY;
          if (mrow[c / TILE]) {
            const float* kc = kb + (int64_t)c * D;
            acc = 0.f;
            for (int d = 0; d < D; ++d) acc += qr[d] * kc[d];
            acc *= sm_scale;
          }
          s[c] = acc;
          if (acc > mx) mx = acc;
        }
        float* orow = o + ((int64_t)bh * N + r) * D;
        for (int d = 0; d < D; ++d) orow[d] = 0.f;
        if (mx == -INFINITY) { if (lse) lse[(int64_t)bh * N + r] = -INFINITY; continue; }
        float den = 0.f;
        for (int c = 0; c < N; ++c) { s[c] = expf(s[c] - mx); den += s[c]; }   /* :39 */
        const float inv = 1.f / den;
        for (int c = 0; c < N; ++c) {                           /* :40 */
          if (s[c] == 0.f) continue;
          const float p = s[c] * inv;
          const float* vc = vb + (int64_t)c * D;
          for (int d = 0; d < D; ++d) orow[d] += p * vc[d];
        }
        if (lse) lse[(int64_t)bh * N + r] = mx + logf(den);
      }
    free(s);
  }
  return 0;
}

static int64_t new_token(int f, int h_, int w, const int dims[3], const int32_t* p) {
  const int c[3] = {f, h_, w};                                  /* permute.py:41-52 */
  return (int64_t)c[p[0]] * (dims[p[1]] * dims[p[2]]) + (int64_t)c[p[1]] * dims[p[2]] + c[p[2]];
}

/* x,out: [BS, NH, T, D] contiguous, esize bytes per element; orders int32 [NH,3]. */
int oracle_reorder(const void* x, void* out, int BS, int NH, int F, int H, int W, int D,
                   int esize, const int32_t* orders) {
  const int T = F * H * W; const int dims[3] = {F, H, W};
  const size_t rowb = (size_t)D * esize;
  for (int b = 0; b < BS; ++b) for (int hd = 0; hd < NH; ++hd) for (int t = 0; t < T; ++t) {
    int f = t / (H * W), t_ = t % (H * W), h_ = t_ / W, w = t_ % W;          /* :27-30 */
    int64_t nt = new_token(f, h_, w, dims, orders + hd * 3);
    const char* src = (const char*)x + (((int64_t)b * NH + hd) * T + t) * rowb;
    char* dst = (char*)out + (((int64_t)b * NH + hd) * T + nt) * rowb;
    memcpy(dst, src, rowb);                                                    /* :54-58 */
  }
  return 0;
}

int oracle_inv_reorder(const void* x, void* out, int BS, int NH, int F, int H, int W, int D,
                       int esize, const int32_t* orders, const int32_t* inv_orders) {
  const int T = F * H * W; const int d0[3] = {F, H, W};
  const size_t rowb = (size_t)D * esize;
  for (int b = 0; b < BS; ++b) for (int hd = 0; hd < NH; ++hd) {
    const int32_t* fp = orders + hd * 3;                                       /* :77-87 */
    const int dims[3] = {d0[fp[0]], d0[fp[1]], d0[fp[2]]};
    for (int t = 0; t < T; ++t) {
      int f = t / (dims[1] * dims[2]), t_ = t % (dims[1] * dims[2]);           /* :90-95 */
      int h_ = t_ / dims[2], w = t_ % dims[2];
      int64_t nt = new_token(f, h_, w, dims, inv_orders + hd * 3);             /* :101-120 */
      const char* src = (const char*)x + (((int64_t)b * NH + hd) * T + t) * rowb;
      char* dst = (char*)out + (((int64_t)b * NH + hd) * T + nt) * rowb;
      memcpy(dst, src, rowb);                                                  /* :122-126 */
    }
  }
  return 0;
}
