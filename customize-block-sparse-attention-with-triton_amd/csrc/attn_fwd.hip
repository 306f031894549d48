// Block-sparse FlashAttention-2 forward for gfx950.
//
// Work decomposition.  The kept tiles of one head form a list in row-major order; it is cut
// into W equal contiguous ranges, one per workgroup, regardless of row boundaries (W depends on
// shapes only, so no host synchronisation on the mask content is needed).  A workgroup walks
// its range row block by row block; the kept tiles of the current row block that fall inside
// the range are split evenly over the workgroup's wavefronts, each of which runs the online
// softmax over its share with private LDS tile buffers, and the per-wavefront results
// (acc, m, l) are merged through LDS.  A row block that lies completely inside the range is
// normalised and written straight to O; a row block shared with a neighbouring workgroup is
// written as an unnormalised partial and merged by combine_kernel.
//
// Per tile a wavefront computes S^T = K Q^T (keys along MFMA rows, queries along lanes), so
// that one lane owns one query: softmax statistics are in-lane reductions plus a single
// cross-half exchange, and P^T leaves the accumulators already in the operand layout of the
// second product O^T += V^T P^T.
//
// Recurrence as the reference kernel, fa2_custom_mask/fa2_fwd.py:146-196 (exp2 domain, fp32
// statistics, P rounded to 16 bits for the second product), with two changes that keep the
// vector ALU out of the way of the matrix cores: the softmax scale is folded into Q, and the
// running maximum is replaced by a reference exponent that is only moved when needed.
#include "common.h"
#include "fwd_split.h"
#include "kernel_util.h"

namespace bsattn {

struct FwdParams {
  const void* q; const void* k; const void* v; void* o; float* lse;
  const int32_t* row_ptr; const int32_t* col_idx;
  float* ws;
  int B, H, N, nb, Bm, Hm, W;   // W: workgroups per head
  int out_f32;
  float qk_scale;  // sm_scale * log2(e)
  int64_t qs[3], ks[3], vs[3], os[3];
};

// P = exp2(score - m) for the 2 x 16 scores one lane holds of one query (key blocks s0, s1),
// rounded to fp16 and packed as the operand fragments pf[0..3][qb] of the second product.
// Returns l + the row sum of the rounded P over this lane's keys.  With FOLD the scores
// already are "scaled score - m".
template <bool FOLD>
__device__ __forceinline__ float softmax_tile(const floatx16& s0, const floatx16& s1, float qk_scale, float m,
                                              float l, uintx4 (&pf)[4][2], int qb) {
  const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
  for (int ts = 0; ts < 4; ++ts) {
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int i = 8 * (ts & 1) + 2 * jj;
      const float x0 = ts < 2 ? s0[i] : s1[i], x1 = ts < 2 ? s0[i + 1] : s1[i + 1];
      const float p0 = __builtin_amdgcn_exp2f(FOLD ? x0 : __builtin_fmaf(x0, qk_scale, -m));
      const float p1 = __builtin_amdgcn_exp2f(FOLD ? x1 : __builtin_fmaf(x1, qk_scale, -m));
      const half2v hp = {(_Float16)p0, (_Float16)p1};
      l = __builtin_amdgcn_fdot2(hp, ones, l, false);
      pf[ts][qb][jj] = __builtin_bit_cast(unsigned int, hp);
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
template <int DB, bool FOLD>
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
  const float delta = fresh ? smax : fmaxf(smax, 0.f);
  m += delta;
  if (!fresh) {
    const float alpha = __builtin_amdgcn_exp2f(-delta);
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

// Number of wavefronts of a workgroup: 2 per SIMD at D=64 (256 VGPRs each), 1 per SIMD at D=128.
template <int D> struct FwdCfg {
  static constexpr int NW = D == 64 ? 8 : 4;
  static constexpr int TILE_BYTES = 64 * 2 * D;             // one K or V tile in LDS
  static constexpr int WAVE_LDS = 2 * TILE_BYTES;           // K buffer + V buffer
  static constexpr int ML_BYTES = NW * 2 * 64 * 4;          // exchange of (m, l) per query
  static constexpr int LDS_BYTES = NW * WAVE_LDS + ML_BYTES;
  static constexpr int R = TILE_BYTES / 256;                // accumulator registers exchanged per round
  static constexpr int ROUNDS = D / R;
  static constexpr int QPW = (R / 4) / NW;                  // output quads per wavefront and round
};

// share of wavefront w in a segment of n tiles starting at a
__device__ __forceinline__ int share_begin(int a, int n, int w, int NW) {
#ifdef EXP_WEIGHTED
  if (NW == 8) { const int cum = w <= 4 ? 3 * w : 12 + 2 * (w - 4); return a + (cum * n) / 20; }
#endif
  return a + (w * n) / NW;
}

template <int D, bool BF16>
__global__ __launch_bounds__(FwdCfg<D>::NW * 64)
void fwd_kernel(const FwdParams prm) {
  using C = FwdCfg<D>;
  constexpr int NW = C::NW;
  constexpr bool FOLD = !BF16;     // fp16: scale folded into Q, reference exponent via an extra MFMA slice
  constexpr int KS = D / 16;       // k-slices of the first product
  constexpr int DB = D / 32;       // 32-wide blocks of the head dimension
  constexpr int CPR = D / 8;       // 16-byte chunks per row
  constexpr int ROWB = 2 * D;      // bytes per LDS row
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

#ifdef EXP_TIMING
  const long long T0 = __builtin_amdgcn_s_memrealtime(); long long Ta = 0, Tb = 0, Tc = 0, Td = 0, Tq = 0; int nseg = 0;
#endif
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ln = lane & 31, g = lane >> 5;
  const int wg = blockIdx.x, bh = blockIdx.y;
  const int b = bh / prm.H, h = bh % prm.H;
  const int mh = (prm.Bm > 1 ? b : 0) * prm.Hm + (prm.Hm > 1 ? h : 0);
  const int nb = prm.nb;
  // the lists are read-only for the whole launch: constant address space => scalar loads
  const cint_ptr_t rp = (cint_ptr_t)(uintptr_t)(prm.row_ptr + (int64_t)mh * nb);
  const cint_ptr_t cols = (cint_ptr_t)(uintptr_t)prm.col_idx;
  const HeadSplit hs = head_split(rp, nb, prm.W, NW);
  if (wg >= hs.Peff) return;
  const int g0 = split_begin(hs, wg), g1 = split_begin(hs, wg + 1);
  if (g0 >= g1) return;

  unsigned char* lds_k = lds + w * C::WAVE_LDS;
  unsigned char* lds_v = lds_k + C::TILE_BYTES;
  float* ml = reinterpret_cast<float*>(lds + NW * C::WAVE_LDS);     // [NW][2][64]
  const unsigned lds_k_addr = (unsigned)(uintptr_t)(lds_ptr_t)lds + w * C::WAVE_LDS;
  const unsigned lds_v_addr = lds_k_addr + C::TILE_BYTES;

  const unsigned short* qg = (const unsigned short*)prm.q + b * prm.qs[0] + h * prm.qs[1];
  const unsigned short* kg = (const unsigned short*)prm.k + b * prm.ks[0] + h * prm.ks[1];
  const unsigned short* vg = (const unsigned short*)prm.v + b * prm.vs[0] + h * prm.vs[1];
  const float qk_scale = prm.qk_scale;

  // per-lane source byte offsets of the asynchronous tile loads (loop invariant)
  unsigned koff[CPR], voff[CPR];
#pragma unroll
  for (int j = 0; j < CPR; ++j) {
    const int c = j * 64 + lane, row = c / CPR, ch = c % CPR;
    koff[j] = 2u * (unsigned)(row * (int)prm.ks[2] + ((ch ^ k_swz<D>(row)) * 8));
    voff[j] = 2u * (unsigned)(row * (int)prm.vs[2] + ((ch ^ v_swz<D>(row)) * 8));
  }
  // per-lane LDS byte offsets of the operand reads.  K fragment (kb, s): row 32kb+ln, chunk 2s+g
  int kaddr[2][KS];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int row = 32 * kb + ln;
      kaddr[kb][s] = row * ROWB + (((2 * s + g) ^ k_swz<D>(row)) * 16);
    }
  // V^T fragment via transpose reads: lane (16-lane block blk, s) supplies 4 halfs of key row
  // 4*(blk/2) + s/4 (+ 16ts + 8jh) at column 16*(blk%2) + 4*(s%4) (+ 32db)
  const int vblk = lane >> 4, vs_ = lane & 15;
  const int vkey0 = 4 * (vblk >> 1) + (vs_ >> 2), vcol0 = 16 * (vblk & 1) + 4 * (vs_ & 3);

  // first row block of the range: largest r with rp[r] <= g0 < rp[r+1]
  int r;
  {
    int lo = 0, hi = nb;  // invariant: rp[lo] <= g0 < rp[hi]
    while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (rp[mid] <= g0) lo = mid; else hi = mid; }
    r = lo;
  }

#ifdef EXP_TIMING
  Ta = __builtin_amdgcn_s_memrealtime();
#endif
  const uintx4 ones_frag = {g == 0 ? 0x3c003c00u : 0u, 0u, 0u, 0u};
  // Asynchronous copies of one wavefront are issued in the order K(j), V(j), K(j'), V(j'), ...
  // (j' the wavefront's next tile): K(j') as soon as the first product of tile j has consumed
  // the K buffer, V(j') as soon as the second product has consumed the V buffer, so every wait
  // below allows exactly the one younger copy (CPR instructions) in flight.  `pre` is the tile
  // whose K copy has been issued ahead (-1: none); its V copy is held back across the merge of
  // a row block, which borrows the V buffers.
  int pre = -1;
  bool first_seg = true;
  int t = g0;
  while (t < g1) {
    const int row_s = rp[r], row_e = rp[r + 1];
    if (row_e <= t) { ++r; continue; }          // row block without kept tiles in the range
    const int seg_a = t, seg_b = row_e < g1 ? row_e : g1, n = seg_b - seg_a;
    const int ma = share_begin(seg_a, n, w, NW), mb = share_begin(seg_a, n, w + 1, NW);
    // this wavefront's first tile in the next segment of the range (-1: none or not adjacent)
    int nxt_seg = -1;
    if (seg_b < g1) {
      int r2 = r + 1;
      while (rp[r2 + 1] <= seg_b) ++r2;
      const int e2 = rp[r2 + 1] < g1 ? rp[r2 + 1] : g1, n2 = e2 - seg_b;
      const int a2 = share_begin(seg_b, n2, w, NW), b2 = share_begin(seg_b, n2, w + 1, NW);
      if (a2 < b2) nxt_seg = a2;
    }

    floatx16 oacc[DB][2];
    float m_i[2] = {0.f, 0.f}, l_i[2] = {0.f, 0.f};
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[db][qb][i] = 0.f;

    if (ma < mb) {
      if (pre != ma) {   // nothing issued ahead for this tile
        const int cb = cols[ma];
        tile_load_async<D>(kg + (int64_t)cb * 64 * prm.ks[2], koff, lds_k_addr);
      }
      tile_load_async<D>(vg + (int64_t)cols[ma] * 64 * prm.vs[2], voff, lds_v_addr);
      // ---- Q fragments (second operand of S^T = K Q^T): lane owns query ln (+32 qb) ----
      uintx4 qf[2][KS];
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        const unsigned short* qrow = qg + (int64_t)(r * 64 + qb * 32 + ln) * prm.qs[2];
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[qb][s] = *reinterpret_cast<const uintx4*>(qrow + 16 * s + 8 * g);
      }
      // vmcnt(0), visible to the compiler: Q is complete here, so that no vector-memory waits
      // of its own end up inside the tile loop (they would also wait for the tile prefetches)
      __builtin_amdgcn_s_waitcnt(0x0F70);
      if constexpr (FOLD) {
        // fold sm_scale*log2(e) into Q once per row block: the scores leave the MFMA already in
        // the exp2 domain (fp16 rounding of the scaled Q perturbs an exponent by ~1e-4)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int s = 0; s < KS; ++s) {
            const uintx4 raw = qf[qb][s];
            const uintx4 scaled = {scale_half2(raw[0], qk_scale), scale_half2(raw[1], qk_scale),
                                   scale_half2(raw[2], qk_scale), scale_half2(raw[3], qk_scale)};
            qf[qb][s] = scaled;
          }
      }
      // m_i: reference exponent of the row (exp2 domain), l_i: per-lane partial sum of P (this
      // lane's half of the keys), both relative to m_i.  m_i starts at 0 and is re-centred on
      // the first tile and whenever a tile produces a P above 2^14.
      // FOLD: "-m_i" enters the scores through one extra contraction slice, ones x (-m_hi, -m_lo)
      uintx4 mfrag[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
      bool fresh = true;
#ifdef EXP_TIMING
      if (nseg == 0) Tq = __builtin_amdgcn_s_memrealtime();
#endif

      for (int j = ma; j < mb; ++j) {
        const int nxt = j + 1 < mb ? j + 1 : nxt_seg;
        const bool has1 = nxt >= 0;
        const int cbn = has1 ? cols[nxt] : 0;

        // ---- S^T[kb][qb] = K[kb] Q[qb]^T (- m_i when FOLD) ----
        // K fragments are read one step ahead of the MFMAs that consume them.
        wait_vm<CPR>();  // K(j) has landed (V(j), issued after it, may still be in flight)
        floatx16 sacc[2][2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int qb = 0; qb < 2; ++qb)
#pragma unroll
            for (int i = 0; i < 16; ++i) sacc[kb][qb][i] = 0.f;
        {
          uintx4 ka[2], kn[2];
#pragma unroll
          for (int kb = 0; kb < 2; ++kb) ka[kb] = *reinterpret_cast<const uintx4*>(lds_k + kaddr[kb][0]);
#pragma unroll
          for (int s = 0; s < KS; ++s) {
            if (s + 1 < KS) {
#pragma unroll
              for (int kb = 0; kb < 2; ++kb) kn[kb] = *reinterpret_cast<const uintx4*>(lds_k + kaddr[kb][s + 1]);
            }
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
              for (int qb = 0; qb < 2; ++qb) sacc[kb][qb] = mfma_qk<BF16>(ka[kb], qf[qb][s], sacc[kb][qb]);
            __builtin_amdgcn_sched_barrier(0);
            if (s + 1 < KS) { ka[0] = kn[0]; ka[1] = kn[1]; }
          }
          if constexpr (FOLD) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
              for (int qb = 0; qb < 2; ++qb) sacc[kb][qb] = mfma_qk<BF16>(ones_frag, mfrag[qb], sacc[kb][qb]);
          }
        }
        // every K fragment has been read: refill the K buffer with the wavefront's next tile
        if (has1) tile_load_async<D>(kg + (int64_t)cbn * 64 * prm.ks[2], koff, lds_k_addr);

        // ---- softmax numerators, one query per lane ----
        // Fast path: P = exp2(score - m_i) with the reference m_i left alone; the row sum of the
        // fp16-rounded P (what the second product consumes) is accumulated with dot2.  If a
        // lane's sum grows by 2^14 or more (or is not finite), some P left the safe fp16 range:
        // recentre() moves m_i to the tile's row maximum and the tile's numerators are redone.
        uintx4 pf[4][2];  // P^T operand fragments: [16-key slice][qb]
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          float lnew = softmax_tile<FOLD>(sacc[0][qb], sacc[1][qb], qk_scale, m_i[qb], l_i[qb], pf, qb);
          if (__any(fresh || !(lnew - l_i[qb] < 16384.0f))) {
            recentre<DB, FOLD>(sacc[0][qb], sacc[1][qb], oacc, qb, qk_scale, m_i[qb], l_i[qb], mfrag[qb], fresh, g);
            lnew = softmax_tile<FOLD>(sacc[0][qb], sacc[1][qb], qk_scale, m_i[qb], l_i[qb], pf, qb);
          }
          l_i[qb] = lnew;
        }
        fresh = false;

        // ---- O^T[db][qb] += V^T[db] P^T[qb]; V^T fragments by LDS transpose reads, one step ahead ----
        if (has1) wait_vm<CPR>(); else wait_vm<0>();  // V(j) has landed (K(nxt) may be in flight)
        {
          auto read_v = [&](int ts, uintx4 (&dst)[DB]) {
#pragma unroll
            for (int db = 0; db < DB; ++db) {
#pragma unroll
              for (int jh = 0; jh < 2; ++jh) {
                const int key = 16 * ts + 8 * jh + vkey0, col = 32 * db + vcol0;
                const int addr = key * ROWB + (((col >> 3) ^ v_swz<D>(key)) * 16) + (col & 7) * 2;
                const short4v rr = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (short4v __attribute__((address_space(3)))*)(lds_v + addr));
                const uintx2 r2 = __builtin_bit_cast(uintx2, rr);
                dst[db][2 * jh] = r2[0]; dst[db][2 * jh + 1] = r2[1];
              }
            }
          };
          uintx4 va[DB], vn[DB];
          read_v(0, va);
#pragma unroll
          for (int ts = 0; ts < 4; ++ts) {
            if (ts + 1 < 4) read_v(ts + 1, vn);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
              uintx4 af = va[db];
              if constexpr (BF16) af = bf16x8_to_f16x8(af);
#pragma unroll
              for (int qb = 0; qb < 2; ++qb)
                oacc[db][qb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, af),
                                                                     __builtin_bit_cast(half8, pf[ts][qb]),
                                                                     oacc[db][qb], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (ts + 1 < 4) {
#pragma unroll
              for (int db = 0; db < DB; ++db) va[db] = vn[db];
            }
          }
        }
        // refill the V buffer, except across the merge below, which borrows it
        if (has1 && j + 1 < mb) tile_load_async<D>(vg + (int64_t)cbn * 64 * prm.vs[2], voff, lds_v_addr);
      }  // tiles of this wavefront
      pre = nxt_seg;
    }

#ifdef EXP_TIMING
    if (nseg == 0) Tb = __builtin_amdgcn_s_memrealtime();
#endif
    // ---- merge the wavefronts' results of this row block through LDS ----
    // Each wavefront publishes (m, l) per query and, round by round, R accumulator registers in
    // its own V buffer ([register][lane] floats); in every round each wavefront reduces QPW
    // groups of 4 registers (4 consecutive head-dimension values of one query per lane) over all
    // contributing wavefronts and writes them out.
    {
      float lsum[2];
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) lsum[qb] = l_i[qb] + __shfl_xor(l_i[qb], 32);
      if (g == 0) {
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          ml[(w * 2 + 0) * 64 + qb * 32 + ln] = ma < mb ? m_i[qb] : -INFINITY;
          ml[(w * 2 + 1) * 64 + qb * 32 + ln] = ma < mb ? lsum[qb] : 0.f;
        }
      }
      const bool full = (seg_a == row_s) && (seg_b == row_e);
      float wgt[NW][2];   // weight of wavefront p's partial for this lane's query of block qb
      float M[2], L[2];
      float* slot = prm.ws + ((((int64_t)bh * prm.W + wg) * 2) + (first_seg ? 0 : 1)) * partial_floats(D);
      void* obase = out_base(prm, b, h);
#pragma unroll
      for (int rd = 0; rd < C::ROUNDS; ++rd) {
        if (ma < mb) {
          float* mine = reinterpret_cast<float*>(lds_v);
#pragma unroll
          for (int e = 0; e < C::R; ++e) {
            const int idx = rd * C::R + e;
            mine[e * 64 + lane] = oacc[idx / 32][(idx / 16) & 1][idx & 15];
          }
        }
        __syncthreads();
        if (rd == 0) {
#pragma unroll
          for (int qb = 0; qb < 2; ++qb) {
            float mm = -INFINITY;
#pragma unroll
            for (int pw = 0; pw < NW; ++pw) mm = fmaxf(mm, ml[(pw * 2 + 0) * 64 + qb * 32 + ln]);
            float ll = 0.f;
#pragma unroll
            for (int pw = 0; pw < NW; ++pw) {
              const float mp = ml[(pw * 2 + 0) * 64 + qb * 32 + ln];
              const float wp = mp == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mp - mm);
              wgt[pw][qb] = wp;
              ll += wp * ml[(pw * 2 + 1) * 64 + qb * 32 + ln];
            }
            M[qb] = mm; L[qb] = ll;
          }
        }
#pragma unroll
        for (int tq = 0; tq < C::QPW; ++tq) {
          const int quad = w * C::QPW + tq;              // group of 4 registers within this round
          const int idx0 = rd * C::R + 4 * quad;         // accumulator register index (db, qb, i16)
          const int db = idx0 / 32, qb = (idx0 / 16) & 1, i4 = (idx0 & 15) / 4;
          float x[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int pw = 0; pw < NW; ++pw) {
            if (share_begin(seg_a, n, pw, NW) < share_begin(seg_a, n, pw + 1, NW)) {   // wavefront pw contributed
              const float* src = reinterpret_cast<const float*>(lds + pw * C::WAVE_LDS + C::TILE_BYTES);
#pragma unroll
              for (int e = 0; e < 4; ++e) x[e] += wgt[pw][qb] * src[(4 * quad + e) * 64 + lane];
            }
          }
          if (full) {
            const float inv = 1.0f / L[qb];
            const int64_t qrow = (int64_t)(r * 64 + qb * 32 + ln);
            store_out4<BF16>(obase, qrow * prm.os[2] + 32 * db + 8 * i4 + 4 * g, prm.out_f32, x[0] * inv, x[1] * inv,
                             x[2] * inv, x[3] * inv);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) slot[(idx0 + e) * 64 + lane] = x[e];
          }
        }
        __syncthreads();
      }
      if (w == 0 && g == 0) {
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          const int64_t qrow = (int64_t)(r * 64 + qb * 32 + ln);
          if (full) {
            if (prm.lse != nullptr)
              prm.lse[((int64_t)bh * prm.N) + qrow] = (M[qb] + __builtin_amdgcn_logf(L[qb])) * 0.6931471805599453f;
          } else {
            slot[64 * D + qb * 32 + ln] = M[qb];
            slot[64 * D + 64 + qb * 32 + ln] = L[qb];
          }
        }
      }
    }
#ifdef EXP_TIMING
    if (nseg == 0) Tc = __builtin_amdgcn_s_memrealtime();
    ++nseg;
#endif
    first_seg = false;
    t = seg_b;
    ++r;
  }
#ifdef EXP_TIMING
  Td = __builtin_amdgcn_s_memrealtime();
  if ((wg % 61) == 5 && lane == 0 && (w == 0 || w == 7))
    printf("wg=%d w=%d tiles=%d segs=%d | setup %lld | Q+first loads %lld | seg0 tiles %lld | seg0 merge %lld | rest %lld | total %lld (x10ns)\n", wg, w, g1 - g0, nseg, Ta - T0, Tq - Ta, Tb - Tq, Tc - Tb, Td - Tc, Td - T0);
#endif
}

// One workgroup per row block: zero-fill empty rows, merge the partials of split rows.
template <int D, bool BF16>
__global__ __launch_bounds__(64) void combine_kernel(const FwdParams prm) {
  constexpr int DB = D / 32;
  const int lane = threadIdx.x, ln = lane & 31, g = lane >> 5;
  const int m = blockIdx.x, bh = blockIdx.y;
  const int b = bh / prm.H, h = bh % prm.H;
  const int mh = (prm.Bm > 1 ? b : 0) * prm.Hm + (prm.Hm > 1 ? h : 0);
  const int nb = prm.nb;
  const int32_t* rp = prm.row_ptr + (int64_t)mh * nb;
  const int rs = rp[m], re = rp[m + 1];
  float acc[DB][2][16];
  float M[2] = {-INFINITY, -INFINITY}, L[2] = {0.f, 0.f};
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[db][qb][i] = 0.f;
  if (re > rs) {
    const HeadSplit hs = head_split(rp, nb, prm.W, FwdCfg<D>::NW);
    const int pf = split_of_tile(hs, rs), pl = split_of_tile(hs, re - 1);
    if (pf == pl) return;  // the whole row lies in one range: already final
    for (int p = pf; p <= pl; ++p) {
      const int pt0 = split_begin(hs, p);
      const int slot_id = (pt0 >= rs) ? 0 : 1;  // is this the first row block of range p?
      const float* slot = prm.ws + ((((int64_t)bh * prm.W + p) * 2) + slot_id) * partial_floats(D);
      float mp[2], lp[2];
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) { mp[qb] = slot[64 * D + qb * 32 + ln]; lp[qb] = slot[64 * D + 64 + qb * 32 + ln]; }
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        const float mn = fmaxf(M[qb], mp[qb]);
        const float so = __builtin_amdgcn_exp2f(M[qb] - mn), sn = __builtin_amdgcn_exp2f(mp[qb] - mn);
        L[qb] = L[qb] * so + lp[qb] * sn;
        M[qb] = mn;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i)
            acc[db][qb][i] = acc[db][qb][i] * so + slot[((db * 2 + qb) * 16 + i) * 64 + lane] * sn;
      }
    }
  }
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const float inv = re > rs ? 1.0f / L[qb] : 0.f;
    const int64_t qrow = (int64_t)(m * 64 + qb * 32 + ln);
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d0 = 32 * db + 8 * i4 + 4 * g;
        float x[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = acc[db][qb][4 * i4 + e] * inv;
        if (prm.out_f32) {
          float* orow = (float*)prm.o + b * prm.os[0] + h * prm.os[1] + qrow * prm.os[2];
          floatx4 w = {x[0], x[1], x[2], x[3]};
          *reinterpret_cast<floatx4*>(orow + d0) = w;
        } else {
          unsigned short* orow = (unsigned short*)prm.o + b * prm.os[0] + h * prm.os[1] + qrow * prm.os[2];
          uintx2 w;
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            if constexpr (BF16) {
              typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
              bf2 hv = {(__bf16)x[2 * e], (__bf16)x[2 * e + 1]};
              w[e] = __builtin_bit_cast(unsigned int, hv);
            } else {
              typedef _Float16 half2v __attribute__((ext_vector_type(2)));
              half2v hv = {(_Float16)x[2 * e], (_Float16)x[2 * e + 1]};
              w[e] = __builtin_bit_cast(unsigned int, hv);
            }
          }
          *reinterpret_cast<uintx2*>(orow + d0) = w;
        }
      }
    if (prm.lse != nullptr && g == 0)
      prm.lse[((int64_t)bh * prm.N) + qrow] =
          re > rs ? (M[qb] + __builtin_amdgcn_logf(L[qb])) * 0.6931471805599453f : -INFINITY;
  }
}

static int groups_per_head(int B, int H, int nb) {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  int64_t W = cus / ((int64_t)B * H);   // one resident workgroup per CU
  const int64_t cap = (int64_t)nb * nb;
  if (W > cap) W = cap;
  if (W < 1) W = 1;
  return (int)W;
}

size_t fwd_workspace_bytes(int B, int H, int N, int D) {
  const int nb = N / 64;
  const int W = groups_per_head(B, H, nb);
  return (size_t)B * H * W * 2 * partial_floats(D) * sizeof(float);
}

template <int D, bool BF16>
static void launch_fwd_t(const FwdParams& prm, int BH, hipStream_t st) {
  using C = FwdCfg<D>;
  static bool configured = false;   // raising the dynamic LDS limit is idempotent
  if (!configured) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&fwd_kernel<D, BF16>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    configured = true;
  }
  hipLaunchKernelGGL((fwd_kernel<D, BF16>), dim3(prm.W, BH), dim3(C::NW * 64), C::LDS_BYTES, st, prm);
  hipLaunchKernelGGL((combine_kernel<D, BF16>), dim3(prm.nb, BH), dim3(64), 0, st, prm);
}

int launch_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
               const int32_t* row_ptr, const int32_t* col_idx, const AttnShape& s, void* ws,
               hipStream_t st) {
  FwdParams prm;
  prm.q = q; prm.k = k; prm.v = v; prm.o = o; prm.lse = lse;
  prm.row_ptr = row_ptr; prm.col_idx = col_idx; prm.ws = (float*)ws;
  prm.B = s.B; prm.H = s.H; prm.N = s.N; prm.nb = s.N / 64; prm.Bm = s.Bm; prm.Hm = s.Hm;
  prm.W = groups_per_head(s.B, s.H, prm.nb);
  prm.out_f32 = s.out_dtype == BSATTN_F32;
  prm.qk_scale = s.sm_scale * 1.4426950408889634f;
  for (int i = 0; i < 3; ++i) { prm.qs[i] = s.qs[i]; prm.ks[i] = s.ks[i]; prm.vs[i] = s.vs[i]; prm.os[i] = s.os[i]; }
  const bool bf = s.dtype == BSATTN_BF16;
  if (s.D == 64 && !bf) launch_fwd_t<64, false>(prm, s.B * s.H, st);
  else if (s.D == 64 && bf) launch_fwd_t<64, true>(prm, s.B * s.H, st);
  else if (s.D == 128 && !bf) launch_fwd_t<128, false>(prm, s.B * s.H, st);
  else launch_fwd_t<128, true>(prm, s.B * s.H, st);
  return launch_status();
}

}  // namespace bsattn
