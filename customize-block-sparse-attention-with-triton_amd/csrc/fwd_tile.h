// Pieces shared by the forward kernels: launch parameters, the softmax of one tile, the rare
// re-centring path.
#pragma once
#include "common.h"
#include "kernel_util.h"

namespace bsattn {

struct FwdParams {
  const void* q; const void* k; const void* v; void* o; float* lse;
  const int32_t* row_ptr; const int32_t* col_idx;
  const unsigned char* tile_partial;        // elementwise masks: per kept tile, 1 = only partly set
  const unsigned long long* tile_bits;      // ... and its 64 row words (bit c = column c)
  float* ws;                       // partial slots of row blocks shared between workgroups (two per workgroup)
  unsigned long long* flags;       // one per row block: parts counted in so far, tagged with `epoch`
  unsigned long long epoch;        // distinguishes this launch's counters from stale contents
  int deterministic;               // tiles go to the wavefronts of a workgroup in a fixed pattern
  int split;                       // pair kernel: workgroups per row block (1: results written directly)
  float* part_o; float* part_ml;   // split > 1: unnormalised fp32 O parts [split][B*H][N][D] and their (m, l) [split][B*H][N][2]
  int B, H, N, nb, Bm, Hm, W;   // W: workgroups per head
  int first_ids;                // workgroups with a linear id below this are the first on their compute unit
  int out_f32;
  float qk_scale;  // sm_scale * log2(e)
  int64_t qs[3], ks[3], vs[3], os[3];
  // fwd_kernel: which range of its head workgroup wg takes, for heads with at least perm_min_tiles kept tiles that
  // are cut into exactly perm_n ranges, the first perm_fast of them with the larger weight (perm_n = 0: none; see
  // range_permutation)
  int perm_n, perm_fast, perm_min_tiles;
  unsigned short perm[512];        // (RANGE_PERM_MAX of range_perm.h)
  unsigned short perm_causal[512]; // the same for heads whose mask is the dense block-causal one
};

// P = exp2(score - m) for the 2 x 16 scores one lane holds of one query (key blocks s0, s1),
// rounded to fp16 and packed as the operand fragments pf[0..3][qb] of the second product.
// Returns l + the row sum of the rounded P over this lane's keys.  With FOLD the scores
// already are "scaled score - m".  PB: P is rounded to bf16 instead of fp16.
template <bool FOLD, bool PB = false>
__device__ __forceinline__ float softmax_tile(const floatx16& s0, const floatx16& s1, float qk_scale, float m,
                                              float l, uintx4 (&pf)[4][2], int qb) {
#pragma unroll
  for (int ts = 0; ts < 4; ++ts) {
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int i = 8 * (ts & 1) + 2 * jj;
      const float x0 = ts < 2 ? s0[i] : s1[i], x1 = ts < 2 ? s0[i + 1] : s1[i + 1];
      const float p0 = __builtin_amdgcn_exp2f(FOLD ? x0 : __builtin_fmaf(x0, qk_scale, -m));
      const float p1 = __builtin_amdgcn_exp2f(FOLD ? x1 : __builtin_fmaf(x1, qk_scale, -m));
      const unsigned int hp = pack2<PB>(p0, p1);
      l = add_packed2<PB>(hp, l);
      pf[ts][qb][jj] = hp;
    }
  }
  return l;
}

__device__ __forceinline__ void* out_base(const FwdParams& prm, int b, int h) {
  const int64_t off = b * prm.os[0] + h * prm.os[1];
  return prm.out_f32 ? (void*)((float*)prm.o + off) : (void*)((unsigned short*)prm.o + off);
}

// Rare path of the softmax: re-centre the reference exponent of one query block on the row
// maximum of the current tile and redo the tile's numerators.
// With elementwise masks (EW) a query may have had nothing but masked keys so far (l == 0, or the
// whole tile masked: maximum -inf): such a lane takes the tile's maximum as its first reference.
template <int DB, bool FOLD, bool EW>
__device__ __forceinline__ void recentre(floatx16& s0, floatx16& s1, floatx16 (&oacc)[DB][2], int qb, float qk_scale,
                                      float& m, float& l, uintx4& mfrag, bool fresh, int g) {
  float mx = max3f(s0[0], s0[1], s0[2]);
#pragma unroll
  for (int i = 3; i < 15; i += 2) mx = max3f(mx, s0[i], s0[i + 1]);
  mx = max3f(mx, s0[15], s1[0]);
#pragma unroll
  for (int i = 1; i < 15; i += 2) mx = max3f(mx, s1[i], s1[i + 1]);
  mx = xhalf_max(fmaxf(mx, s1[15]));
  // exponent of the largest entry relative to the current reference
  const float smax = FOLD ? mx : __builtin_fmaf(mx, qk_scale, -m);
  float delta = fresh ? smax : fmaxf(smax, 0.f);
  bool nomass = false;
  if constexpr (EW) {
    // (a query's keys are split over two lanes, which must keep one common reference: the mass is
    // the sum of both halves, or a lane whose own keys were all masked would drift away)
    nomass = !fresh && l + __shfl_xor(l, 32) == 0.f;
    if (nomass) delta = smax;
    if (smax == -INFINITY) delta = 0.f;
  }
  m += delta;
  if (!fresh) {
    const float alpha = nomass ? 1.0f : __builtin_amdgcn_exp2f(-delta);
    l *= alpha;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[db][qb][i] *= alpha;
  }
  if constexpr (FOLD) {
#pragma unroll
    for (int i = 0; i < 16; ++i) { s0[i] -= delta; s1[i] -= delta; }
    const _Float16 hi = (_Float16)(-m);
    const _Float16 lo = (_Float16)(-m - (float)hi);
    const half2v hl = {hi, lo};
    mfrag[0] = g == 0 ? __builtin_bit_cast(unsigned int, hl) : 0u;
  }
}


}  // namespace bsattn
