/* Runs every function of the C oracle (oracle/bsattn_oracle.c) on small seeded inputs, edge cases
 * included, in a build with the address and undefined-behaviour sanitizers: any out-of-bounds access or
 * undefined operation aborts the program.  The values themselves are checked by the Python tests. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

int oracle_build_groups(const uint8_t* mask, int B, int H, int nb, int32_t* groups, int32_t* n_list,
                        int64_t* G_out, int64_t* T_out);
int oracle_naive_fwd(const float* q, const float* k, const float* v, const uint8_t* mask, int BH, int BHm, int N, int D,
                     float sm_scale, int row0, int row1, float* o, float* lse);
int oracle_reorder(const void* x, void* out, int BS, int NH, int F, int Hh, int W, int D, int elem_bytes,
                   const int32_t* orders);
int oracle_inv_reorder(const void* x, void* out, int BS, int NH, int F, int Hh, int W, int D, int elem_bytes,
                       const int32_t* orders, const int32_t* inv_orders);

static uint64_t state = 0x9E3779B97F4A7C15ull;
static uint32_t rnd(void) { state ^= state << 13; state ^= state >> 7; state ^= state << 17; return (uint32_t)(state >> 16); }
static float frand(void) { return (float)(rnd() % 2001) / 1000.0f - 1.0f; }

int main(void) {
  /* kept-tile groups: empty masks, full masks, random ones */
  for (int it = 0; it < 60; ++it) {
    const int B = 1 + rnd() % 2, H = 1 + rnd() % 3, nb = 1 + rnd() % 9;
    const int keep = it % 3 == 0 ? 0 : (it % 3 == 1 ? 100 : (int)(rnd() % 100));
    uint8_t* mask = malloc((size_t)B * H * nb * nb);
    for (int i = 0; i < B * H * nb * nb; ++i) mask[i] = (int)(rnd() % 100) < keep;
    int32_t* groups = malloc(sizeof(int32_t) * B * H * nb * 5);
    int32_t* n_list = malloc(sizeof(int32_t) * (B * H * nb * nb > 0 ? B * H * nb * nb : 1));
    int64_t G = -1, T = -1;
    if (oracle_build_groups(mask, B, H, nb, groups, n_list, &G, &T) != 0 || G < 0 || T < 0) { printf("groups\n"); return 1; }
    free(mask); free(groups); free(n_list);
  }
  /* naive attention: shared and per-head masks, rows without keys, a row range */
  for (int it = 0; it < 12; ++it) {
    const int B = 1 + it % 2, H = 1 + it % 3, nb = 1 + it % 4, N = 64 * nb, D = it % 2 ? 64 : 16;
    const int BHm = it % 2 ? B * H : 1;
    const size_t n = (size_t)B * H * N * D;
    float *q = malloc(4 * n), *k = malloc(4 * n), *v = malloc(4 * n), *o = malloc(4 * n), *lse = malloc(4 * (size_t)B * H * N);
    for (size_t i = 0; i < n; ++i) { q[i] = frand(); k[i] = frand(); v[i] = frand(); }
    uint8_t* mask = malloc((size_t)BHm * nb * nb);
    for (int i = 0; i < BHm * nb * nb; ++i) mask[i] = rnd() % 3 != 0;
    for (int c = 0; c < nb; ++c) mask[c] = 0;                       /* first row block keeps nothing */
    const int row0 = it % 4 == 3 ? 32 : 0, row1 = it % 4 == 3 ? N - 16 : N;
    if (oracle_naive_fwd(q, k, v, mask, B * H, BHm, N, D, 0.125f, row0, row1, o, it % 5 == 4 ? NULL : lse) != 0) { printf("fwd\n"); return 1; }
    free(q); free(k); free(v); free(o); free(lse); free(mask);
  }
  /* reorder and its inverse: every permutation, 2- and 4-byte elements, the round trip is the identity */
  static const int32_t perms[6][3] = {{0, 1, 2}, {0, 2, 1}, {1, 2, 0}, {1, 0, 2}, {2, 1, 0}, {2, 0, 1}};
  static const int32_t inv[6][3] = {{0, 1, 2}, {0, 2, 1}, {2, 0, 1}, {1, 0, 2}, {2, 1, 0}, {1, 2, 0}};
  for (int it = 0; it < 12; ++it) {
    const int BS = 1 + it % 2, NH = 6, F = 2 + it % 3, Hh = 3, W = 4 + it % 2, D = 8, eb = it % 2 ? 4 : 2;
    const size_t bytes = (size_t)BS * NH * F * Hh * W * D * eb;
    unsigned char *x = malloc(bytes), *y = malloc(bytes), *z = malloc(bytes);
    for (size_t i = 0; i < bytes; ++i) x[i] = (unsigned char)rnd();
    int32_t orders[18], inv_orders[18];
    for (int h = 0; h < NH; ++h) for (int j = 0; j < 3; ++j) { orders[3 * h + j] = perms[(h + it) % 6][j]; inv_orders[3 * h + j] = inv[(h + it) % 6][j]; }
    if (oracle_reorder(x, y, BS, NH, F, Hh, W, D, eb, orders) != 0) { printf("reorder\n"); return 1; }
    if (oracle_inv_reorder(y, z, BS, NH, F, Hh, W, D, eb, orders, inv_orders) != 0) { printf("inv_reorder\n"); return 1; }
    for (size_t i = 0; i < bytes; ++i) if (x[i] != z[i]) { printf("round trip\n"); return 1; }
    free(x); free(y); free(z);
  }
  printf("ok\n");
  return 0;
}
