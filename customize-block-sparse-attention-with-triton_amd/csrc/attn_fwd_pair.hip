// Block-sparse FlashAttention-2 forward, head dimension 128 for launches with many row blocks, and
// head dimension 256 (the only forward kernel for it; one wavefront per SIMD there, K and V fragments
// taken from LDS in two portions).
//
// At D = 128 a wavefront that owns 64 queries needs all 512 registers of its SIMD, so the
// general kernel (attn_fwd.hip) runs one wavefront per SIMD and is bound by instruction issue.
// Here a row block belongs to a pair of wavefronts, 32 queries each (256 registers: two
// wavefronts per SIMD), which share one K and one V tile buffer: a workgroup is one pair, four
// workgroups fit a compute unit, and the grid has one workgroup per (head, row block) - the
// hardware's dispatcher balances the load, no merge is ever needed.  Heads are taken in groups
// of 8, head i of a group on XCD i (workgroups go to XCDs round-robin by linear id), so that the
// row blocks resident on an XCD share one head's K and V in its L2; long row blocks of
// block-causal masks come first.
//
// Tile arithmetic, softmax and layouts are those of attn_fwd.hip (fa2_custom_mask/fa2_fwd.py:146-196
// of the reference), with a single block of 32 queries per wavefront.
#include "common.h"
#include "fwd_tile.h"
#include "kernel_util.h"

namespace bsattn {

constexpr int PAIR_EARLY_V = 1;   // largest number of fragment portions (head dimension / 128) for which V is read early
constexpr int PAIR_COLS_CAP = 1024;                               // column indices of the row block kept in LDS
template <int D> constexpr int pair_lds_bytes() { return 2 * 64 * 2 * D + 512 + PAIR_COLS_CAP * 4; }   // K tile, V tile, mask words, columns

// CONTIG: the rows of K and of V follow each other without gaps (row stride = D).
template <int D, int DT, bool EW, bool CONTIG>
__global__ __launch_bounds__(128, D == 128 ? 2 : 1) void fwd_pair_kernel(const FwdParams prm) {
  constexpr int KS = D / 16, DB = D / 32, CPR = D / 8, ROWB = 2 * D, TILE_BYTES = 64 * ROWB;
  constexpr int PORTIONS = D / 128;              // K and V fragments are read in this many portions
  constexpr int KSP = KS / PORTIONS, DBP = DB / PORTIONS;
  constexpr bool BF16 = DT != 0;
  constexpr bool PB = DT == 2;                   // P rounded to bf16, second product in bf16 (V as it is)
  constexpr bool FOLD = !BF16;
  constexpr int HALF = CPR / 2;                  // copy instructions per wavefront and tile
  constexpr int KOPS = HALF + (EW ? 1 : 0), VOPS = HALF;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ln = lane & 31, g = lane >> 5;
  const int nb = prm.nb, BH = prm.B * prm.H;
  // linear id -> (head, row block): groups of 8 heads, one head per XCD, long row blocks first
  int bh, m;
  const int per_chunk = gridDim.x / prm.split;    // chunk = slowest index: head i of a group stays on XCD i
  const int chunk = blockIdx.x / per_chunk;
  {
    const int L = blockIdx.x - chunk * per_chunk;
    const int grp = L / (8 * nb), l = L - grp * 8 * nb;
    const int hg = BH - 8 * grp < 8 ? BH - 8 * grp : 8;
    bh = 8 * grp + l % hg;
    m = nb - 1 - l / hg;
    if (m < 0) return;                           // padding of an incomplete last group
  }
  const int b = bh / prm.H, h = bh % prm.H;
  const int mh = (prm.Bm > 1 ? b : 0) * prm.Hm + (prm.Hm > 1 ? h : 0);
  const cint_ptr_t rp = (cint_ptr_t)(uintptr_t)(prm.row_ptr + (int64_t)mh * nb);
  // Q of this lane's query (second operand of S^T = K Q^T) depends on the block index only: asked for first, it
  // travels while the list is looked up and the first tiles are requested.
  const int64_t qrow = (int64_t)m * 64 + 32 * w + ln;          // this lane's query
  uintx4 qf[1][KS];
  {
    const unsigned short* qp = (const unsigned short*)prm.q + b * prm.qs[0] + h * prm.qs[1] + qrow * prm.qs[2];
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[0][s] = *reinterpret_cast<const uintx4*>(qp + 16 * s + 8 * g);
  }
  int t0 = rp[m], t1 = rp[m + 1];
  if (prm.split > 1) {                           // this workgroup's share of the row block's list
    const int len = t1 - t0;
    t1 = t0 + (int)((int64_t)len * (chunk + 1) / prm.split);
    t0 = t0 + (int)((int64_t)len * chunk / prm.split);
    if (t0 == t1) return;                        // (pair_sum_parts_kernel knows which shares are empty)
  }
  void* obase = out_base(prm, b, h);
  if (t0 == t1) {                                // no kept tile: O = 0, lse = -inf
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
        store_out4<BF16>(obase, qrow * prm.os[2] + 32 * db + 8 * i4 + 4 * g, prm.out_f32, 0.f, 0.f, 0.f, 0.f);
    if (prm.lse != nullptr && g == 0) prm.lse[(int64_t)bh * prm.N + qrow] = -INFINITY;
    return;
  }

  unsigned char* lds_k = lds;
  unsigned char* lds_v = lds + TILE_BYTES;
  const unsigned long long* lds_bits = reinterpret_cast<const unsigned long long*>(lds + 2 * TILE_BYTES);
  int* lcols = reinterpret_cast<int*>(lds + 2 * TILE_BYTES + 512);
  const unsigned lds_k_addr = (unsigned)(uintptr_t)(lds_ptr_t)lds;
  const unsigned lds_v_addr = lds_k_addr + TILE_BYTES;
  const unsigned lds_bits_addr = lds_k_addr + 2 * TILE_BYTES;

  const unsigned short* kg = (const unsigned short*)prm.k + b * prm.ks[0] + h * prm.ks[1];
  const unsigned short* vg = (const unsigned short*)prm.v + b * prm.vs[0] + h * prm.vs[1];
  const float qk_scale = prm.qk_scale;

  // column indices of the row block (EW: "partly set" in bit 30), staged once
  const cint_ptr_t cols = (cint_ptr_t)(uintptr_t)prm.col_idx;
  typedef const unsigned char __attribute__((address_space(4)))* cbyte_ptr_t;
  auto flagged_col = [&](int t) {
    int c = cols[t];
    if constexpr (EW) c |= (int)((cbyte_ptr_t)(uintptr_t)prm.tile_partial)[t] << 30;
    return c;
  };
  constexpr int COL_MASK = 0x3fffffff;
  auto col_of = [&](int t) { return t - t0 < PAIR_COLS_CAP ? lcols[t - t0] : flagged_col(t); };

  // asynchronous tile copies: copy instruction j covers tile rows [4j, 4j+4); this wavefront issues
  // the instructions [HALF w, HALF (w+1)) of every tile (and 256 of the 512 bytes of mask words)
  // (the swizzles repeat every 16 rows for K and every 4 rows for V: KPER / VPER instructions)
  constexpr int RPI = 64 / CPR, KPER = 16 / RPI, VPER = RPI >= 4 ? 1 : 4 / RPI;
  unsigned koff[KPER], voff[VPER];
  {
    const int row0 = lane / CPR, ch = lane % CPR;
#pragma unroll
    for (int par = 0; par < KPER; ++par)
      koff[par] = 2u * (unsigned)(row0 * (int)prm.ks[2] + ((ch ^ k_swz<D>(par * RPI + row0)) * 8));
#pragma unroll
    for (int par = 0; par < VPER; ++par)
      voff[par] = 2u * (unsigned)(row0 * (int)prm.vs[2] + ((ch ^ v_swz<D>(par * RPI + row0)) * 8));
  }
  const int64_t k_rs = CONTIG ? (int64_t)D : prm.ks[2], v_rs = CONTIG ? (int64_t)D : prm.vs[2];   // row strides
  auto k_copy = [&](int cb, int t) {
    const unsigned short* tile = kg + (int64_t)cb * 64 * k_rs;
    if constexpr (CONTIG) {     // (instruction j reads at byte 1024 j of the tile and writes at byte 1024 j of the buffer)
#pragma unroll
      for (int jb = 0; jb < HALF; jb += 4)
        tile_load_async_four(tile + (w * HALF + jb) * RPI * D, koff[jb % KPER], koff[(jb + 1) % KPER], koff[(jb + 2) % KPER],
                             koff[(jb + 3) % KPER], lds_k_addr + (w * HALF + jb) * 1024);
    } else {
#pragma unroll
      for (int jj = 0; jj < HALF; ++jj) {
        const int j = w * HALF + jj;
        tile_load_async_one(tile + (int64_t)j * RPI * k_rs, koff[jj % KPER], lds_k_addr + j * 1024);
      }
    }
    if constexpr (EW) {
      const unsigned long long* src = prm.tile_bits + (int64_t)t * 64;
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2"
                   :: "s"(lds_bits_addr + w * 256), "v"(4u * (unsigned)lane + 256u * w), "s"(src) : "memory", "m0");
    }
  };
  auto v_copy = [&](int cb) {
    const unsigned short* tile = vg + (int64_t)cb * 64 * v_rs;
    if constexpr (CONTIG) {
#pragma unroll
      for (int jb = 0; jb < HALF; jb += 4)
        tile_load_async_four(tile + (w * HALF + jb) * RPI * D, voff[jb % VPER], voff[(jb + 1) % VPER], voff[(jb + 2) % VPER],
                             voff[(jb + 3) % VPER], lds_v_addr + (w * HALF + jb) * 1024);
    } else {
#pragma unroll
      for (int jj = 0; jj < HALF; ++jj) {
        const int j = w * HALF + jj;
        tile_load_async_one(tile + (int64_t)j * RPI * v_rs, voff[jj % VPER], lds_v_addr + j * 1024);
      }
    }
  };
  static_assert(HALF % KPER == 0 && HALF % VPER == 0, "the swizzle patterns of a wavefront's instructions start at phase 0");

  // fragment addresses (as in attn_fwd.hip)
  int kaddr[2][KS];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int row = 32 * kb + ln;
      kaddr[kb][s] = row * ROWB + (((2 * s + g) ^ k_swz<D>(row)) * 16);
    }
  const int vblk = lane >> 4, vs_ = lane & 15;
  const int vkey0 = 4 * (vblk >> 1) + (vs_ >> 2), vcol0 = 16 * (vblk & 1) + 4 * (vs_ & 3);
  const uintx4 ones_frag = {g == 0 ? 0x3c003c00u : 0u, 0u, 0u, 0u};

  // first tile's copies (its column from one scalar load), then the column list into LDS
  int cx = flagged_col(t0);
  k_copy(cx & COL_MASK, t0);
  v_copy(cx & COL_MASK);
  for (int i = threadIdx.x; i < t1 - t0 && i < PAIR_COLS_CAP; i += 128) {
    int c = prm.col_idx[t0 + i];
    if constexpr (EW) c |= (int)prm.tile_partial[t0 + i] << 30;
    lcols[i] = c;
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);               // vmcnt(0), visible to the compiler: Q and the first tiles
  if constexpr (FOLD) {
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const uintx4 raw = qf[0][s];
      const uintx4 scaled = {scale_half2(raw[0], qk_scale), scale_half2(raw[1], qk_scale),
                             scale_half2(raw[2], qk_scale), scale_half2(raw[3], qk_scale)};
      qf[0][s] = scaled;
    }
  }
  floatx16 oacc[DB][2];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) { oacc[db][0][i] = 0.f; oacc[db][1][i] = 0.f; }
  float m_i = 0.f, l_i = 0.f;
  uintx4 mfrag = {0u, 0u, 0u, 0u};
  bool fresh = true;
  int any_m = 0;     // (wave-uniform) some lane's reference exponent is not zero: the extra contraction slice is needed
  __syncthreads();                                  // both halves of K(t0) and V(t0) and the column list are in LDS

  for (int t = t0; t < t1; ++t) {
    const bool has1 = t + 1 < t1;
    const int cxn = has1 ? __builtin_amdgcn_readfirstlane(col_of(t + 1)) : 0;
    const bool partial = EW && (cx >> 30) != 0;
    // ---- S^T = K Q^T (- m when FOLD); the K fragments (and the mask word of this lane's query) ----
    floatx16 s0, s1;
#pragma unroll
    for (int i = 0; i < 16; ++i) { s0[i] = 0.f; s1[i] = 0.f; }
    unsigned long long mw = 0ull;
#pragma unroll
    for (int pt = 0; pt < PORTIONS; ++pt) {
      uintx4 kfr[2][KSP];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int s = 0; s < KSP; ++s) kfr[kb][s] = *reinterpret_cast<const uintx4*>(lds_k + kaddr[kb][pt * KSP + s]);
      if (pt == PORTIONS - 1) {
        if constexpr (EW) { if (partial) mw = lds_bits[32 * w + ln] >> (4 * g); }
        lds_wait();
        __syncthreads();                            // both wavefronts hold their K fragments: the K buffer is free
        if (has1) k_copy(cxn & COL_MASK, t + 1);
      }
#pragma unroll
      for (int s = 0; s < KSP; ++s) {
        s0 = mfma_qk<BF16>(kfr[0][s], qf[0][pt * KSP + s], s0);
        s1 = mfma_qk<BF16>(kfr[1][s], qf[0][pt * KSP + s], s1);
      }
    }
    if constexpr (FOLD) {
      if (any_m) {
        s0 = mfma_qk<BF16>(ones_frag, mfrag, s0);
        s1 = mfma_qk<BF16>(ones_frag, mfrag, s1);
      }
    }
    if constexpr (EW) {
      if (partial) {
        const unsigned lo = (unsigned)mw, hi = (unsigned)(mw >> 32);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const unsigned bit = 1u << (8 * (i / 4) + (i % 4));
          s0[i] = (lo & bit) ? s0[i] : -INFINITY;
          s1[i] = (hi & bit) ? s1[i] : -INFINITY;
        }
      }
    }
    uintx4 pf[4][2];
    // ---- V^T fragments ----
    auto v_landed = [&]() {
      if (has1) wait_vm<KOPS>(); else wait_vm<0>();   // this wavefront's half of V(t) has landed (K(t+1) may be in flight)
      if (t > t0) __syncthreads();                    // ... and the other half (the first tile was waited for above)
    };
    auto read_v = [&](int pt, uintx4 (&vfr)[4][DBP]) {
#pragma unroll
      for (int ts = 0; ts < 4; ++ts)
#pragma unroll
        for (int db = 0; db < DBP; ++db) {
          uintx4 a;
#pragma unroll
          for (int jh = 0; jh < 2; ++jh) {
            const int key = 16 * ts + 8 * jh + vkey0, col = 32 * (pt * DBP + db) + vcol0;
            const int addr = key * ROWB + (((col >> 3) ^ v_swz<D>(key)) * 16) + (col & 7) * 2;
            const short4v rr = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (short4v __attribute__((address_space(3)))*)(lds_v + addr));
            const uintx2 r2 = __builtin_bit_cast(uintx2, rr);
            a[2 * jh] = r2[0]; a[2 * jh + 1] = r2[1];
          }
          if constexpr (BF16 && !PB) a = bf16x8_to_f16x8(a);
          vfr[ts][db] = a;
        }
    };
    auto v_free = [&]() {
      lds_wait();
      __syncthreads();                            // both wavefronts hold their V fragments: the V buffer is free
      if (has1) v_copy(cxn & COL_MASK);
    };
    auto second = [&](int pt, uintx4 (&vfr)[4][DBP]) {
#pragma unroll
      for (int ts = 0; ts < 4; ++ts)
#pragma unroll
        for (int db = 0; db < DBP; ++db)
          oacc[pt * DBP + db][0] = mfma_qk<PB>(vfr[ts][db], pf[ts][0], oacc[pt * DBP + db][0]);
    };
    auto numerators = [&]() {
      float lnew = softmax_tile<FOLD, PB>(s0, s1, qk_scale, m_i, l_i, pf, 0);
      // (FOLD: the first tile of a row block keeps the reference at 0 when its sums are of moderate size)
      const bool first = FOLD ? fresh && !(lnew >= 0.25f) : fresh;
      if (__any(first || (EW && l_i == 0.f) || !(lnew - l_i < 16384.0f))) {
        recentre<DB, FOLD, EW>(s0, s1, oacc, 0, qk_scale, m_i, l_i, mfrag, fresh, g);
        any_m = 1;
        lnew = softmax_tile<FOLD, PB>(s0, s1, qk_scale, m_i, l_i, pf, 0);
      }
      l_i = lnew;
      fresh = false;
    };
    if constexpr (PORTIONS <= PAIR_EARLY_V) {
      // The V fragments are read before the softmax (they take the registers of the K fragments), so
      // that the next V tile is requested that much earlier: its latency was exposed otherwise.
      uintx4 vfr[PORTIONS][4][DBP];
      v_landed();
#pragma unroll
      for (int pt = 0; pt < PORTIONS; ++pt) read_v(pt, vfr[pt]);
      v_free();
      numerators();
#pragma unroll
      for (int pt = 0; pt < PORTIONS; ++pt) second(pt, vfr[pt]);
    } else {
      numerators();
      v_landed();
      // ---- O^T += V^T P^T, the V^T fragments taken in PORTIONS portions ----
#pragma unroll
      for (int pt = 0; pt < PORTIONS; ++pt) {
        uintx4 vfr[4][DBP];
        read_v(pt, vfr);
        if (pt == PORTIONS - 1) v_free();
        second(pt, vfr);
      }
    }
    if (has1) {
      wait_vm<VOPS>();                              // this wavefront's half of K(t+1) has landed (V(t+1) may be in flight)
      __syncthreads();                              // ... and the other half
    }
    cx = cxn;
  }

  // ---- normalise and write ----
  const float lsum = l_i + __shfl_xor(l_i, 32);
  if (prm.split > 1) {   // unnormalised fp32 part with its reference exponent and row sum
    float* part = prm.part_o + ((int64_t)chunk * BH + bh) * prm.N * D;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
        store_out4<BF16>(part, qrow * D + 32 * db + 8 * i4 + 4 * g, true, oacc[db][0][4 * i4], oacc[db][0][4 * i4 + 1],
                         oacc[db][0][4 * i4 + 2], oacc[db][0][4 * i4 + 3]);
    if (g == 0) {
      float* ml = prm.part_ml + (((int64_t)chunk * BH + bh) * prm.N + qrow) * 2;
      ml[0] = m_i; ml[1] = lsum;
    }
    return;
  }
  const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
  // the wavefront's 32 rows of O leave through its half of the (now idle) LDS
  static_assert(2 * rows_out_bytes(D, true) <= pair_lds_bytes<D>(), "room for the result rows of both wavefronts");
  __syncthreads();           // the other wavefront has left its last tile
  rows_out<BF16, D>(lds + w * rows_out_bytes(D, true), obase, ((int64_t)m * 64 + 32 * w) * prm.os[2], prm.os[2], prm.out_f32,
                    lane, [&](int db, int i) { return oacc[db][0][i] * inv; });
  if (prm.lse != nullptr && g == 0)
    prm.lse[(int64_t)bh * prm.N + qrow] =
        lsum > 0.f ? (m_i + __builtin_amdgcn_logf(lsum)) * 0.6931471805599453f : -INFINITY;
}

// split > 1: O = sum_c 2^(m_c - M) O_c / sum_c 2^(m_c - M) l_c over the non-empty shares c of a row block
// (M = max m_c over shares with mass), lse = (M + log2 of the denominator) ln 2.  One thread per 4
// consecutive output values.
template <bool BF16>
__global__ __launch_bounds__(256) void pair_sum_parts_kernel(const FwdParams prm, int D, int64_t quads) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= quads) return;
  const int qpr = D / 4;                                     // threads per query row
  const int64_t rowg = i / qpr;                              // row over all heads
  const int col = (int)(i % qpr) * 4;
  const int bh = (int)(rowg / prm.N), row = (int)(rowg % prm.N);
  const int b = bh / prm.H, h = bh % prm.H, BH = prm.B * prm.H;
  const int mh = (prm.Bm > 1 ? b : 0) * prm.Hm + (prm.Hm > 1 ? h : 0);
  const int32_t* rp = prm.row_ptr + (int64_t)mh * prm.nb;
  const int t0 = rp[row / 64], len = rp[row / 64 + 1] - t0;
  float M = -INFINITY;
  for (int c = 0; c < prm.split; ++c) {
    if ((int64_t)len * c / prm.split == (int64_t)len * (c + 1) / prm.split) continue;      // empty share: nothing was written
    const float* ml = prm.part_ml + (((int64_t)c * BH + bh) * prm.N + row) * 2;
    if (ml[1] > 0.f) M = fmaxf(M, ml[0]);
  }
  float L = 0.f;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int c = 0; c < prm.split; ++c) {
    if ((int64_t)len * c / prm.split == (int64_t)len * (c + 1) / prm.split) continue;
    const float* ml = prm.part_ml + (((int64_t)c * BH + bh) * prm.N + row) * 2;
    if (!(ml[1] > 0.f)) continue;
    const float wgt = __builtin_amdgcn_exp2f(ml[0] - M);
    L += wgt * ml[1];
    acc += wgt * *reinterpret_cast<const floatx4*>(prm.part_o + (((int64_t)c * BH + bh) * prm.N + row) * D + col);
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  store_out4<BF16>(out_base(prm, b, h), (int64_t)row * prm.os[2] + col, prm.out_f32, acc[0] * inv, acc[1] * inv, acc[2] * inv,
                   acc[3] * inv);
  if (col == 0 && prm.lse != nullptr)
    prm.lse[(int64_t)bh * prm.N + row] = L > 0.f ? (M + __builtin_amdgcn_logf(L)) * 0.6931471805599453f : -INFINITY;
}

template <int D, int DT, bool EW, bool CONTIG>
static void launch_pair_c(const FwdParams& prm, int grid, hipStream_t st) {
  static std::atomic<unsigned long long> configured{0};   // raising the dynamic LDS limit is idempotent
  once_per_device(configured, [] {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&fwd_pair_kernel<D, DT, EW, CONTIG>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, pair_lds_bytes<D>());
  });
  hipLaunchKernelGGL((fwd_pair_kernel<D, DT, EW, CONTIG>), dim3(grid), dim3(128), pair_lds_bytes<D>(), st, prm);
}

template <int D, int DT, bool EW>
static void launch_pair_t(const FwdParams& prm, hipStream_t st) {
  const int BH = prm.B * prm.H;
  const int grid = ((BH + 7) / 8) * 8 * prm.nb * prm.split;
  // (the variant with immediate copy offsets: 5 % faster at D = 256, 3 % slower on dense masks at D = 128)
  if (D == 256 && prm.ks[2] == D && prm.vs[2] == D) launch_pair_c<D, DT, EW, D == 256>(prm, grid, st);
  else launch_pair_c<D, DT, EW, false>(prm, grid, st);
  if (prm.split > 1) {
    const int64_t quads = (int64_t)BH * prm.N * D / 4;
    hipLaunchKernelGGL((pair_sum_parts_kernel<DT != 0>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, st, prm, D, quads);
  }
}

template <int D>
static void launch_pair_d(const FwdParams& prm, int dt, bool elementwise, hipStream_t st) {
  if (!elementwise) {
    if (dt == 0) launch_pair_t<D, 0, false>(prm, st);
    else if (dt == 1) launch_pair_t<D, 1, false>(prm, st);
    else launch_pair_t<D, 2, false>(prm, st);
  } else {
    if (dt == 0) launch_pair_t<D, 0, true>(prm, st);
    else if (dt == 1) launch_pair_t<D, 1, true>(prm, st);
    else launch_pair_t<D, 2, true>(prm, st);
  }
}

// D: 128 or 256.  dt: 0 fp16, 1 bf16 with P rounded to fp16 (V converted), 2 bf16 with P rounded to bf16.
void launch_fwd_pair(const FwdParams& prm, int D, int dt, bool elementwise, hipStream_t st) {
  if (D == 128) launch_pair_d<128>(prm, dt, elementwise, st);
  else launch_pair_d<256>(prm, dt, elementwise, st);
}

}  // namespace bsattn
