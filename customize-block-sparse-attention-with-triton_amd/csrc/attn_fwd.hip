// Block-sparse FlashAttention-2 forward for gfx950.
//
// Work decomposition: every wavefront is an independent worker (one 64-thread workgroup).
// The kept tiles of one head form a list in row-major order; it is cut into `P` equal
// contiguous ranges, one per wavefront, regardless of row boundaries.  A wavefront walks
// its range row block by row block.  A row block that lies completely inside the range is
// normalised and written straight to O; a row block shared with a neighbouring range is
// written as an unnormalised partial (acc, m, l) and merged by combine_kernel.  The grid
// depends on shapes only, so no host synchronisation on the mask content is needed.
//
// Per tile the wavefront computes S^T = K Q^T (keys along MFMA rows, queries along lanes),
// so that one lane owns one query: the online-softmax row maximum and sum are in-lane
// reductions plus a single cross-half exchange, and P^T leaves the accumulators already in
// the operand layout of the second product O^T += V^T P^T.
//
// Recurrence as the reference kernel: fa2_custom_mask/fa2_fwd.py:146-196 (exp2 domain,
// l summed in fp32 before P is rounded).
#include "common.h"
#include "fwd_split.h"
#ifdef EXP_ENV_P
#include <cstdlib>
#endif

namespace bsattn {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));
typedef unsigned int uintx2 __attribute__((ext_vector_type(2)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));

struct FwdParams {
  const void* q; const void* k; const void* v; void* o; float* lse;
  const int32_t* row_ptr; const int32_t* col_idx;
  float* ws;
  int B, H, N, nb, Bm, Hm, P;
  int out_f32;
  float qk_scale;  // sm_scale * log2(e)
  int64_t qs[3], ks[3], vs[3], os[3];
};

__device__ __forceinline__ void wave_lds_sync() {
  // LDS regions are private to a wavefront; order its own writes before its reads.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ float max3f(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

__device__ __forceinline__ float xhalf_max(float x) {
  // max of lane l and lane l^32 (the two halves of a wavefront hold the same query)
  return fmaxf(x, __shfl_xor(x, 32));
}

template <bool BF16>
__device__ __forceinline__ floatx16 mfma_qk(uintx4 a, uintx4 b, floatx16 c) {
  if constexpr (BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a),
                                                  __builtin_bit_cast(half8, b), c, 0, 0, 0);
}

// two packed fp16 values times an fp32 scalar, rounded back to fp16
__device__ __forceinline__ unsigned int scale_half2(unsigned int x, float c) {
  const half2v h = __builtin_bit_cast(half2v, x);
  const half2v r = {(_Float16)((float)h[0] * c), (_Float16)((float)h[1] * c)};
  return __builtin_bit_cast(unsigned int, r);
}

// bf16 bits -> fp16 bits, 8 at a time (exact for the magnitudes attention inputs take)
__device__ __forceinline__ uintx4 bf16x8_to_f16x8(uintx4 x) {
  uintx4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float lo = __builtin_bit_cast(float, x[i] << 16);
    const float hi = __builtin_bit_cast(float, x[i] & 0xffff0000u);
    half2v h = {(_Float16)lo, (_Float16)hi};
    r[i] = __builtin_bit_cast(unsigned int, h);
  }
  return r;
}

// 16-byte chunk swizzles of the LDS tiles (rows of D halfs = D/8 chunks).
//  K tile: operand reads take one chunk of 32 consecutive rows -> spread the chunk index over rows.
//  V tile: transpose reads take 64 contiguous bytes of 4 consecutive rows -> move rows to
//          different 64-byte parts of the 256-byte bank period.
template <int D> __device__ __forceinline__ int k_swz(int row) { return D == 64 ? ((row >> 1) & 7) : (row & 15); }
template <int D> __device__ __forceinline__ int v_swz(int row) { return D == 64 ? (((row >> 1) & 1) << 2) : ((row & 3) << 2); }

typedef unsigned char __attribute__((address_space(3)))* lds_ptr_t;
typedef const int32_t __attribute__((address_space(4)))* cint_ptr_t;

// Asynchronous global -> LDS copy of one 64 x D tile: D/8 instructions, each moving 16 bytes
// per lane; the data of lane l lands at lds + j*1024 + l*16.  `off` holds the per-lane
// source byte offsets from `tile` (a wave-uniform base).  The copies are issued from
// inline assembly so that the compiler's own wait-count insertion does not serialise
// them; completion is awaited explicitly with wait_vm<N>() (vector memory operations
// retire in order, so "at most N outstanding" means everything older than the N youngest
// has landed).
template <int D>
__device__ __forceinline__ void tile_load_async(const unsigned short* tile, const unsigned (&off)[D / 8],
                                                unsigned lds_addr) {
#ifdef EXP_NOLOAD
  return;
#endif
#pragma unroll
  for (int j = 0; j < D / 8; ++j)
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_addr + j * 1024), "v"(off[j]), "s"(tile) : "memory", "m0");
}


template <int N> __device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}

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

__device__ __forceinline__ void lds_wait() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// 4 consecutive output values of one row: fp32, or packed fp16/bf16
template <bool BF16>
__device__ __forceinline__ void store_out4(void* obase, int64_t elem_off, bool out_f32, float x0, float x1,
                                           float x2, float x3) {
  if (out_f32) {
    const floatx4 w = {x0, x1, x2, x3};
    *reinterpret_cast<floatx4*>((float*)obase + elem_off) = w;
  } else {
    uintx2 w;
    if constexpr (BF16) {
      typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
      const bf2 a = {(__bf16)x0, (__bf16)x1}, c = {(__bf16)x2, (__bf16)x3};
      w[0] = __builtin_bit_cast(unsigned int, a); w[1] = __builtin_bit_cast(unsigned int, c);
    } else {
      const half2v a = {(_Float16)x0, (_Float16)x1}, c = {(_Float16)x2, (_Float16)x3};
      w[0] = __builtin_bit_cast(unsigned int, a); w[1] = __builtin_bit_cast(unsigned int, c);
    }
    *reinterpret_cast<uintx2*>((unsigned short*)obase + elem_off) = w;
  }
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

template <int D, bool BF16>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(D == 64 ? 2 : 1)))
void fwd_kernel(const FwdParams prm) {
  constexpr bool FOLD = !BF16;     // fp16: scale folded into Q, reference exponent via an extra MFMA slice
  constexpr int KS = D / 16;       // k-slices of the first product
  constexpr int DB = D / 32;       // 32-wide blocks of the head dimension
  constexpr int CPR = D / 8;       // 16-byte chunks per row
  constexpr int ROWB = 2 * D;      // bytes per LDS row
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k[64 * ROWB];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v[64 * ROWB];

#ifdef EXP_TIMING
  const long long T0 = __builtin_amdgcn_s_memrealtime(); long long T1 = 0, T2 = 0, T3 = 0, T4 = 0; int nseg = 0;
#endif
  const int lane = threadIdx.x;
  const int ln = lane & 31, g = lane >> 5;
  const int p = blockIdx.x, bh = blockIdx.y;
  const int b = bh / prm.H, h = bh % prm.H;
  const int mh = (prm.Bm > 1 ? b : 0) * prm.Hm + (prm.Hm > 1 ? h : 0);
  const int nb = prm.nb;
  // the lists are read-only for the whole launch: constant address space => scalar loads
  const cint_ptr_t rp = (cint_ptr_t)(uintptr_t)(prm.row_ptr + (int64_t)mh * nb);
  const cint_ptr_t cols = (cint_ptr_t)(uintptr_t)prm.col_idx;
  const HeadSplit hs = head_split(rp, nb, prm.P);
  if (p >= hs.Peff) return;
  const int t0 = split_begin(hs, p), t1 = split_begin(hs, p + 1);
  if (t0 >= t1) return;

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
  const unsigned lds_k_addr = (unsigned)(uintptr_t)(lds_ptr_t)lds_k;
  const unsigned lds_v_addr = (unsigned)(uintptr_t)(lds_ptr_t)lds_v;
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

  // Tiles j of this wavefront's range are processed in order.  Asynchronous copies are issued
  // in the order K(j), V(j), K(j+1), V(j+1), ...: K(j+1) as soon as the first product of tile j
  // has consumed the K buffer, V(j+1) as soon as the second product has consumed the V buffer,
  // so every wait below allows exactly the one younger copy (CPR instructions) in flight.
  {
    const int cb = cols[t0];
    tile_load_async<D>(kg + (int64_t)cb * 64 * prm.ks[2], koff, lds_k_addr);
    tile_load_async<D>(vg + (int64_t)cb * 64 * prm.vs[2], voff, lds_v_addr);
  }

  // first row block of the range: largest r with rp[r] <= t0 < rp[r+1]
  int r;
  {
    int lo = 0, hi = nb;  // invariant: rp[lo] <= t0 < rp[hi]
    while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (rp[mid] <= t0) lo = mid; else hi = mid; }
    r = lo;
  }

#ifdef EXP_TIMING
  T1 = __builtin_amdgcn_s_memrealtime();
#endif
  // state of the current row block
  uintx4 qf[2][KS];
  floatx16 oacc[DB][2];
  // m_i: reference exponent of the row (exp2 domain), l_i: per-lane partial sum of P (this
  // lane's half of the keys), both relative to m_i.  m_i starts at 0 and is re-centred on the
  // first tile and whenever a tile produces a P above 2^14.
  float m_i[2], l_i[2];
  // FOLD: "-m_i" enters the scores through one extra contraction slice, ones x (-m_hi, -m_lo)
  uintx4 mfrag[2];
  const uintx4 ones_frag = {g == 0 ? 0x3c003c00u : 0u, 0u, 0u, 0u};
  bool fresh = true, seg_begin = true, first_seg = true;
  int seg_t = t0, seg_end = t0, row_s = 0, row_e = 0;

  for (int j = t0; j < t1; ++j) {
    if (seg_begin) {
      while (rp[r + 1] <= j) ++r;      // skip row blocks without kept tiles
      row_s = rp[r]; row_e = rp[r + 1];
      seg_t = j; seg_end = row_e < t1 ? row_e : t1;
      // ---- Q fragments (second operand of S^T = K Q^T): lane owns query ln (+32 qb) ----
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
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int i = 0; i < 16; ++i) oacc[db][qb][i] = 0.f;
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        m_i[qb] = 0.f; l_i[qb] = 0.f;
        mfrag[qb] = uintx4{0u, 0u, 0u, 0u};
      }
      fresh = true;
      seg_begin = false;
#ifdef EXP_TIMING
      if (nseg == 0) T2 = __builtin_amdgcn_s_memrealtime();
      ++nseg;
#endif
    }
    const bool has1 = j + 1 < t1;
    const int cbn = has1 ? cols[j + 1] : 0;

    // ---- S^T[kb][qb] = K[kb] Q[qb]^T (- m_i when FOLD) ----
    // K fragments are read one step ahead of the MFMAs that consume them.
    wait_vm<CPR>();  // K(j) has landed (V(j), issued after it, may still be in flight)
#ifdef EXP_PRIO
    __builtin_amdgcn_s_setprio(EXP_PRIO);
#endif
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
#ifdef EXP_PRIO
    __builtin_amdgcn_s_setprio(0);
#endif
    // every K fragment has been read: refill the K buffer with the next tile
    if (has1) tile_load_async<D>(kg + (int64_t)cbn * 64 * prm.ks[2], koff, lds_k_addr);

    // ---- softmax numerators, one query per lane ----
    // Fast path: P = exp2(score - m_i) with the reference m_i left alone; the row sum of the
    // fp16-rounded P (what the second product consumes) is accumulated with dot2.  If a lane's
    // sum grows by 2^14 or more (or is not finite), some P left the safe fp16 range: recentre()
    // moves m_i to the tile's row maximum and the tile's numerators are redone.
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
    if (has1) wait_vm<CPR>(); else wait_vm<0>();  // V(j) has landed (K(j+1) may be in flight)
#ifdef EXP_PRIO
    __builtin_amdgcn_s_setprio(EXP_PRIO);
#endif
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
#ifdef EXP_PRIO
    __builtin_amdgcn_s_setprio(0);
#endif
    if (has1) tile_load_async<D>(vg + (int64_t)cbn * 64 * prm.vs[2], voff, lds_v_addr);

#ifdef EXP_TIMING
    if (j == t0) T3 = __builtin_amdgcn_s_memrealtime();
#endif
    if (j + 1 == seg_end) {
      // ---- epilogue of the row block ----
      const bool full = (seg_t == row_s) && (seg_end == row_e);
      float lsum[2];
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) lsum[qb] = l_i[qb] + __shfl_xor(l_i[qb], 32);
      if (full) {
        void* obase = out_base(prm, b, h);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          const float inv = 1.0f / lsum[qb];
          const int64_t qrow = (int64_t)(r * 64 + qb * 32 + ln);
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4)
              store_out4<BF16>(obase, qrow * prm.os[2] + 32 * db + 8 * i4 + 4 * g, prm.out_f32,
                               oacc[db][qb][4 * i4] * inv, oacc[db][qb][4 * i4 + 1] * inv,
                               oacc[db][qb][4 * i4 + 2] * inv, oacc[db][qb][4 * i4 + 3] * inv);
          if (prm.lse != nullptr && g == 0)
            prm.lse[((int64_t)bh * prm.N) + qrow] = (m_i[qb] + __builtin_amdgcn_logf(lsum[qb])) * 0.6931471805599453f;
        }
      } else {
        // partial slot: [acc index][lane] floats, then m[64], l[64]
        float* slot = prm.ws + ((((int64_t)bh * prm.P + p) * 2) + (first_seg ? 0 : 1)) * partial_floats(D);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int qb = 0; qb < 2; ++qb)
#pragma unroll
            for (int i = 0; i < 16; ++i) slot[((db * 2 + qb) * 16 + i) * 64 + lane] = oacc[db][qb][i];
        if (g == 0) {
#pragma unroll
          for (int qb = 0; qb < 2; ++qb) {
            slot[64 * D + qb * 32 + ln] = m_i[qb];
            slot[64 * D + 64 + qb * 32 + ln] = lsum[qb];
          }
        }
      }
      first_seg = false;
      seg_begin = true;
      ++r;
    }
  }
#ifdef EXP_TIMING
  T4 = __builtin_amdgcn_s_memrealtime();
  if ((p % 293) == 5 && lane == 0)
    printf("p=%d tiles=%d segs=%d | setup %lld | Qload+init %lld | first tile %lld | rest %lld | total %lld (x10ns) start@%lld\n", p, t1 - t0, nseg, T1 - T0, T2 - T1, T3 - T2, T4 - T3, T4 - T0, T0 % 100000);
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
    const HeadSplit hs = head_split(rp, nb, prm.P);
    const int pf = split_of_tile(hs, rs), pl = split_of_tile(hs, re - 1);
    if (pf == pl) return;  // the whole row lies in one range: already final
    for (int p = pf; p <= pl; ++p) {
      const int pt0 = split_begin(hs, p);
      const int slot_id = (pt0 >= rs) ? 0 : 1;  // is this the first row block of range p?
      const float* slot = prm.ws + ((((int64_t)bh * prm.P + p) * 2) + slot_id) * partial_floats(D);
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

static int waves_per_head(int B, int H, int nb) {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
#ifdef EXP_ENV_P
  if (getenv("BSATTN_P")) return atoi(getenv("BSATTN_P"));
#endif
  const int64_t target = (int64_t)cus * 8;  // one resident round: 2 wavefronts per SIMD
  int64_t P = (target + (int64_t)B * H - 1) / ((int64_t)B * H);
  const int64_t cap = (int64_t)nb * nb;
  if (P > cap) P = cap;
  if (P < 1) P = 1;
  return (int)P;
}

size_t fwd_workspace_bytes(int B, int H, int N, int D) {
  const int nb = N / 64;
  const int P = waves_per_head(B, H, nb);
  return (size_t)B * H * P * 2 * partial_floats(D) * sizeof(float);
}

int launch_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
               const int32_t* row_ptr, const int32_t* col_idx, const AttnShape& s, void* ws,
               hipStream_t st) {
  FwdParams prm;
  prm.q = q; prm.k = k; prm.v = v; prm.o = o; prm.lse = lse;
  prm.row_ptr = row_ptr; prm.col_idx = col_idx; prm.ws = (float*)ws;
  prm.B = s.B; prm.H = s.H; prm.N = s.N; prm.nb = s.N / 64; prm.Bm = s.Bm; prm.Hm = s.Hm;
  prm.P = waves_per_head(s.B, s.H, prm.nb);
  prm.out_f32 = s.out_dtype == BSATTN_F32;
  prm.qk_scale = s.sm_scale * 1.4426950408889634f;
  for (int i = 0; i < 3; ++i) { prm.qs[i] = s.qs[i]; prm.ks[i] = s.ks[i]; prm.vs[i] = s.vs[i]; prm.os[i] = s.os[i]; }
  const dim3 grid(prm.P, s.B * s.H), cgrid(prm.nb, s.B * s.H);
  const bool bf = s.dtype == BSATTN_BF16;
  if (s.D == 64 && !bf) {
    hipLaunchKernelGGL((fwd_kernel<64, false>), grid, dim3(64), 0, st, prm);
    hipLaunchKernelGGL((combine_kernel<64, false>), cgrid, dim3(64), 0, st, prm);
  } else if (s.D == 64 && bf) {
    hipLaunchKernelGGL((fwd_kernel<64, true>), grid, dim3(64), 0, st, prm);
    hipLaunchKernelGGL((combine_kernel<64, true>), cgrid, dim3(64), 0, st, prm);
  } else if (s.D == 128 && !bf) {
    hipLaunchKernelGGL((fwd_kernel<128, false>), grid, dim3(64), 0, st, prm);
    hipLaunchKernelGGL((combine_kernel<128, false>), cgrid, dim3(64), 0, st, prm);
  } else {
    hipLaunchKernelGGL((fwd_kernel<128, true>), grid, dim3(64), 0, st, prm);
    hipLaunchKernelGGL((combine_kernel<128, true>), cgrid, dim3(64), 0, st, prm);
  }
  return launch_status();
}

}  // namespace bsattn
