// Block-sparse FlashAttention-2 forward for gfx950.
//
// Work decomposition.  The kept tiles of one head form a list in row-major order; it is cut
// into W contiguous ranges, one per workgroup, regardless of row boundaries (W depends on
// shapes only, so no host synchronisation on the mask content is needed; where two workgroups
// share a compute unit the first-comer's range is longer, see fwd_split.h).  A workgroup walks
// its range row block by row block; the kept tiles of the current row block that fall inside
// the range are handed to the workgroup's wavefronts one at a time, each wavefront runs the
// online softmax over the tiles it gets with private LDS tile buffers, and the per-wavefront
// results (acc, m, l) are merged through LDS.  A row block that lies completely inside the
// range is normalised and written straight to O.  A row block cut by range boundaries is
// finished by the workgroup that holds its first tiles: the others publish unnormalised parts
// in the workspace (device-scope stores, then a flag), and it pulls them when it gets there.
// With many row blocks per workgroup (many heads) each wavefront takes whole row blocks
// instead, and nothing is merged.
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
#include <atomic>
#include <mutex>
#include <map>
#include <array>
#include <chrono>
#include <cstdlib>
#include "common.h"
#include "fwd_split.h"
#include "fwd_tile.h"
#include "kernel_util.h"
#include "range_perm.h"

namespace bsattn {

// A workgroup is four wavefronts, one per SIMD.  At D=64 a wavefront needs 256 registers and two
// workgroups share a compute unit (while one merges or waits for its first tiles the other computes);
// at D=128 a wavefront needs all 512 registers of its SIMD.
template <int D> struct FwdCfg {
  static constexpr int NW = 4;
  static constexpr int WG_PER_CU = D == 64 ? 2 : 1;
  static constexpr int TILE_BYTES = 64 * 2 * D;             // one K or V tile in LDS
  static constexpr int WAVE_LDS = 2 * TILE_BYTES;           // K buffer + V buffer
  static constexpr int ML_BYTES = NW * 2 * 64 * 4 + 64;     // exchange of (m, l) per query + the tile counter
  static constexpr int COLS_CAP = 2048;                     // column indices of the range kept in LDS
  static constexpr int BITS_OFF = NW * WAVE_LDS + ML_BYTES + COLS_CAP * 4;   // mask words of the current tile, 512 bytes per wavefront
  static constexpr int LDS_BYTES = BITS_OFF + NW * 512;
  static constexpr int R = WAVE_LDS / 256;                  // accumulator registers exchanged per round (K and V buffer)
  static constexpr int ROUNDS = D / R;
  static constexpr int QPW = (R / 4) / NW;                  // output quads per wavefront and round
  static constexpr int SHORT_ROW = 6 * NW;                  // row blocks up to this many tiles may go to one wavefront
  static constexpr int SNAP = WG_PER_CU > 1 ? 16 : 8;       // short ranges: a boundary at least this close to an end of its row block moves there
};

// DT: 0 fp16; 1 bf16 with P rounded to fp16 (V fragments converted); 2 bf16 with P rounded to bf16.
// CONTIG: the rows of K and of V follow each other without gaps (row stride = D).
template <int D, int DT, bool ROWS, bool EW, bool CONTIG>
__global__ __launch_bounds__(FwdCfg<D>::NW * 64, FwdCfg<D>::WG_PER_CU)
void fwd_kernel(const FwdParams prm) {
  constexpr bool BF16 = DT != 0, PB = DT == 2;
  using C = FwdCfg<D>;
  constexpr int NW = C::NW;
  constexpr bool FOLD = !BF16;     // fp16: scale folded into Q, reference exponent via an extra MFMA slice
  constexpr int KS = D / 16;       // k-slices of the first product
  constexpr int DB = D / 32;       // 32-wide blocks of the head dimension
  constexpr int CPR = D / 8;       // 16-byte chunks per row
  constexpr int ROWB = 2 * D;      // bytes per LDS row
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ln = lane & 31, g = lane >> 5;
  // linear id -> (head, range): heads interleaved, so that every head gets its share of the
  // workgroups that are first on their compute unit
  const int BH = prm.B * prm.H;
  const int bh = blockIdx.x % BH;
  int wg = blockIdx.x / BH;
  const int b = bh / prm.H, h = bh % prm.H;
  const int mh = (prm.Bm > 1 ? b : 0) * prm.Hm + (prm.Hm > 1 ? h : 0);
  const int nb = prm.nb;
  // the lists are read-only for the whole launch: constant address space => scalar loads
  const cint_ptr_t rp = (cint_ptr_t)(uintptr_t)(prm.row_ptr + (int64_t)mh * nb);
  const cint_ptr_t cols = (cint_ptr_t)(uintptr_t)prm.col_idx;
  HeadSplit hs = head_split(rp, nb, prm.W, /*min_tiles=*/NW, prm.first_ids > bh ? (prm.first_ids - bh + BH - 1) / BH : 0, 0);
  // Long ranges (the regime of the weighted shares) are cut on the axis with gaps and boundaries move to a row
  // block's end only from very close; short ranges are cut on the plain tile axis and their boundaries move to
  // the nearer end of a row block from up to half a range (and at least SNAP tiles) away: a row block is shared
  // only where a boundary falls into its middle, row blocks of up to a range's length or 2 SNAP tiles never (N = 17536,
  // one head, against 8 tiles for every head: keep 0.15 36.0 -> 31.4 us, keep 0.2 40.0 -> 34.6, keep 0.25 43.2 -> 39.8,
  // keep 0.05 21.8 -> 20.2, keep 0.1 25.8 -> 25.1; keep 0.35 and above, other sizes: +-1 %).
  constexpr int LONG_GAP = 12, LONG_SNAP = 2;
  const bool long_ranges = !ROWS && ((int64_t)hs.T >= (int64_t)EQUAL_SPLIT_BELOW * hs.Peff || hs.Peff >= 3 * nb);   // (or row blocks much longer than the ranges)
  // (D = 128, one workgroup per compute unit and tiles twice as long: sharing a row block is cheaper against the
  // imbalance it avoids; 8 tiles for every head.  Half a range there: keep 0.1 87 -> 98 us, keep 0.15 107 -> 129 us.)
  const int half_range = hs.T / (2 * (hs.Peff > 0 ? hs.Peff : 1)) + 1;
  // (long ranges over short row blocks, up to 32 tiles on average: a boundary moves to the nearer end of its row block
  // from up to half such a row block away, so that next to no row block is shared; against 2 tiles: 8 heads of
  // N = 17536 at keep 0.05 67.9 -> 62 us, 4 heads at keep 0.1 57.9 -> 54.6 us; with longer row blocks the imbalance
  // costs more than the sharing: keep 0.35, one head, 48.0 -> 50.4 us with 12 tiles)
  const int avg_row = hs.T / (nb > 0 ? nb : 1);
  const int long_snap = avg_row <= 32 ? avg_row / 2 + 1 : LONG_SNAP;
  const int snap = long_ranges ? long_snap : (C::WG_PER_CU > 1 && half_range > C::SNAP ? half_range : C::SNAP);
  // (ranges that are long only against the row blocks they lie in, several to a row block: 24 positions; N = 6400
  // dense 31.2 -> 29.0 us, where 12 are best for N = 17536 dense, 102.1 against 104.0 us)
  const int long_gap = (int64_t)hs.T >= (int64_t)EQUAL_SPLIT_BELOW * hs.Peff ? LONG_GAP : 2 * LONG_GAP;
  if (long_ranges) { hs.gap = long_gap; hs.X = (int64_t)hs.T + (int64_t)long_gap * nb; }
  // Which range this workgroup takes (launches with few heads and long ranges): the ranges of a head start at
  // all phases of a row, and workgroups that share an XCD, hence an L2, get ranges of like phase, so that they
  // walk the same column blocks at the same time (dense N = 17536, one head: 42 instead of 196 MB fetched from
  // HBM per launch, 104.5 instead of 106.6 us).  The phases are those of rows of equal length: heads that keep less
  // than three quarters of their tiles are left alone (keep 0.5 measured 2 % slower with the permutation), except
  // the dense block-causal mask, which has a table of its own (N = 32000: 185 instead of 193 us).
  if (prm.perm_n > 0 && prm.perm_n == hs.Peff && prm.perm_fast == hs.fast) {
    if (hs.T >= prm.perm_min_tiles) wg = prm.perm[wg];
    // the dense block-causal mask (by its number of kept tiles and the length of one row in the middle; a mask
    // taken for it by mistake merely gets its ranges in another order): ranges sorted by their first column block
    else if ((int64_t)hs.T * 2 == (int64_t)nb * (nb + 1) && rp[nb / 2 + 1] - rp[nb / 2] == nb / 2 + 1) wg = prm.perm_causal[wg];
  }
  // Heads cut into equal shares: the two workgroups of a compute unit (linear ids L and L + first_ids: the
  // dispatcher places them in the same order in both rounds) take neighbouring ranges 2k and 2k + 1.  A boundary that
  // moves to a row block's end moves tiles from one range to its neighbour; between the two workgroups of a compute
  // unit that changes nothing in what the compute unit has to do, and only every other boundary unbalances the
  // compute units (keep 0.1, N = 17536: 26.2 -> 24.8 us; keep 0.25: 42.2 -> 41.6 us).  (All boundaries move by the
  // same rule: one that may move further than its neighbours can overtake them.)
  {
    const int Fh = prm.first_ids > bh ? (prm.first_ids - bh + BH - 1) / BH : 0;
    if (!ROWS && hs.fast == 0 && hs.Peff == prm.W && prm.W == 2 * Fh) wg = wg < Fh ? 2 * wg : 2 * (wg - Fh) + 1;
  }
  // Row blocks without kept tiles belong to no range: they are dealt round-robin over all workgroups
  // of the head, which write O = 0, lse = -inf for their share.  (With whole row blocks per
  // wavefront the ranges are row-aligned and cover them, unless the head keeps nothing at all.)
  if (!ROWS || hs.T == 0) {
    for (int r0 = wg; r0 < nb; r0 += prm.W) {
      if (rp[r0 + 1] > rp[r0]) continue;
      void* ob = out_base(prm, b, h);
      for (int i = threadIdx.x; i < 64 * (D / 4); i += NW * 64) {
        const int64_t qrow = (int64_t)r0 * 64 + i / (D / 4);
        store_out4<BF16>(ob, qrow * prm.os[2] + 4 * (i % (D / 4)), prm.out_f32, 0.f, 0.f, 0.f, 0.f);
      }
      if (prm.lse != nullptr && threadIdx.x < 64) prm.lse[(int64_t)bh * prm.N + (int64_t)r0 * 64 + threadIdx.x] = -INFINITY;
    }
  }
  if (hs.T == 0 || wg >= hs.Peff) return;
  // where the range begins and ends on the cutting axis (ROWS: the plain tile axis, as absolute tile offsets)
  const int64_t x0 = split_pos(hs, wg), x1 = split_pos(hs, wg + 1);
  int g0 = hs.lo + (int)x0, g1 = hs.lo + (int)x1;     // (ROWS; the other mode finds its tiles below)
  if constexpr (!ROWS) {
    if (x0 >= x1) return;
  }

  unsigned char* lds_k = lds + w * C::WAVE_LDS;
  unsigned char* lds_v = lds_k + C::TILE_BYTES;
  float* ml = reinterpret_cast<float*>(lds + NW * C::WAVE_LDS);     // [NW][2][64]
  const unsigned lds_k_addr = (unsigned)(uintptr_t)(lds_ptr_t)lds + w * C::WAVE_LDS;
  const unsigned lds_v_addr = lds_k_addr + C::TILE_BYTES;

  const unsigned short* qg = (const unsigned short*)prm.q + b * prm.qs[0] + h * prm.qs[1];
  const unsigned short* kg = (const unsigned short*)prm.k + b * prm.ks[0] + h * prm.ks[1];
  const unsigned short* vg = (const unsigned short*)prm.v + b * prm.vs[0] + h * prm.vs[1];
  const float qk_scale = prm.qk_scale;

  // Per-lane source byte offsets of the asynchronous tile loads (loop invariant).  Copy
  // instruction j covers rows [64j/CPR, 64(j+1)/CPR) of the tile; the row part of the offset is
  // added to the (scalar) tile pointer, the per-lane part only depends on j through the chunk
  // swizzle, whose pattern repeats with period KPER in j (K) or not at all (V).
  constexpr int RPI = 64 / CPR;                 // tile rows per copy instruction
  constexpr int KPER = D == 64 ? 2 : 4;         // period of the K swizzle in copy instructions
  unsigned koff[KPER], voff[1];
  {
    const int row0 = lane / CPR, ch = lane % CPR;
#pragma unroll
    for (int par = 0; par < KPER; ++par)
      koff[par] = 2u * (unsigned)(row0 * (int)prm.ks[2] + ((ch ^ k_swz<D>(par * RPI + row0)) * 8));
    voff[0] = 2u * (unsigned)(row0 * (int)prm.vs[2] + ((ch ^ v_swz<D>(row0)) * 8));
  }
  static_assert(D == 64 || D == 128, "swizzle periods below are derived for 64 and 128");
  auto k_copy = [&](const unsigned short* tile, int j) {
    tile_load_async_one(tile + (int64_t)j * RPI * prm.ks[2], koff[j % KPER], lds_k_addr + j * 1024);
  };
  auto v_copy = [&](const unsigned short* tile, int j) {
    tile_load_async_one(tile + (int64_t)j * RPI * prm.vs[2], voff[0], lds_v_addr + j * 1024);
  };
  const unsigned lds_bits_addr = (unsigned)(uintptr_t)(lds_ptr_t)lds + C::BITS_OFF + w * 512;
  const unsigned long long* lds_bits = reinterpret_cast<const unsigned long long*>(lds + C::BITS_OFF + w * 512);
  constexpr int KOPS = CPR + (EW ? 2 : 0);      // instructions of one K copy
  // copy of the K tile `tile` = entry t of the kept-tile list (EW: with its 512 bytes of mask words)
  // CONTIG (rows that follow each other without gaps, the usual case): copy instruction j reads at
  // byte offset 1024 j from the tile and writes at 1024 j from the buffer, and the instruction's immediate
  // offset applies to both, so four instructions share one scalar base and one m0 (6 instead of 24 scalar
  // instructions per tile copy at D = 64).
  constexpr bool k_contig = CONTIG, v_contig = CONTIG;
  const int64_t k_rs = CONTIG ? (int64_t)D : prm.ks[2], v_rs = CONTIG ? (int64_t)D : prm.vs[2];   // row strides (a constant: a tile's address is a shift)
  auto k_copy_all = [&](const unsigned short* tile, int t) {
    if constexpr (k_contig) {
#pragma unroll
      for (int jb = 0; jb < CPR; jb += 4)
        tile_load_async_four(tile + jb * RPI * D, koff[jb % KPER], koff[(jb + 1) % KPER], koff[(jb + 2) % KPER], koff[(jb + 3) % KPER],
              lds_k_addr + jb * 1024);
    } else {
#pragma unroll
      for (int j = 0; j < CPR; ++j) k_copy(tile, j);
    }
    if constexpr (EW) {
      const unsigned long long* src = prm.tile_bits + (int64_t)t * 64;
#pragma unroll
      for (int j = 0; j < 2; ++j)
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2"
                     :: "s"(lds_bits_addr + j * 256), "v"(4u * (unsigned)lane + 256u * j), "s"(src) : "memory", "m0");
    }
  };
  auto v_copy_all = [&](const unsigned short* tile) {
    if constexpr (v_contig) {
#pragma unroll
      for (int jb = 0; jb < CPR; jb += 4)
        tile_load_async_four(tile + jb * RPI * D, voff[0], voff[0], voff[0], voff[0], lds_v_addr + jb * 1024);
    } else {
#pragma unroll
      for (int j = 0; j < CPR; ++j) v_copy(tile, j);
    }
  };
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

  const uintx4 ones_frag = {g == 0 ? 0x3c003c00u : 0u, 0u, 0u, 0u};

  // ---- state of the row block a wavefront is working on, and the steps both drivers share ----
  uintx4 qf[2][KS];          // Q fragments (second operand of S^T = K Q^T): lane owns query ln (+32 qb)
  floatx16 oacc[DB][2];
  // m_i: reference exponent of the row (exp2 domain), l_i: per-lane partial sum of P (this lane's
  // half of the keys), both relative to m_i.  m_i starts at 0 and is re-centred on the first tile
  // and whenever a tile produces a P above 2^14.
  float m_i[2], l_i[2];
  // FOLD: "-m_i" enters the scores through one extra contraction slice, ones x (-m_hi, -m_lo)
  uintx4 mfrag[2];
  bool fresh = true;
  int any_m = 0;     // (wave-uniform) some lane's reference exponent is not zero: the extra contraction slice is needed

  auto reset_acc = [&]() {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[db][qb][i] = 0.f;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) { m_i[qb] = 0.f; l_i[qb] = 0.f; mfrag[qb] = uintx4{0u, 0u, 0u, 0u}; }
    fresh = true;
    any_m = 0;
  };
  auto load_q = [&](int r) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const unsigned short* qrow = qg + (int64_t)(r * 64 + qb * 32 + ln) * prm.qs[2];
#pragma unroll
      for (int s = 0; s < KS; ++s) qf[qb][s] = *reinterpret_cast<const uintx4*>(qrow + 16 * s + 8 * g);
    }
    // vmcnt(0), visible to the compiler: Q is complete here, so that no vector-memory waits of
    // its own end up inside the tile loop (they would also wait for the tile prefetches)
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
  };

  // One 64 x 64 tile whose K and V copies have been issued (K first).  has1: the wavefront has a
  // next tile, in column block cbn, whose K copy is issued as soon as this tile's K fragments sit
  // in registers; copy_v: its V copy may be issued too, as soon as this tile's V fragments sit in
  // registers.  Copies are therefore issued in the order K(cur), V(cur), K(nxt), V(nxt), ..., and
  // every wait allows exactly the one younger copy (CPR instructions) in flight.  `mid` runs once
  // the first LDS wait of the tile has passed (the place to pick up earlier LDS results).
  // The tile is processed as four blocks so that the matrix cores and the vector ALU of this
  // wavefront overlap: [1] scores of query block 0, [2] scores of query block 1 interleaved with
  // the softmax numerators of block 0, [3] second product of block 0 interleaved with the
  // numerators of block 1, [4] second product of block 1.  Operand fragments are read from LDS
  // once, all at once (the read latency is a multiple of an MFMA's issue interval), and serve
  // both query blocks.
  auto tile = [&](bool has1, int cbn, int tn, bool copy_v, bool partial, auto&& mid) {
    // D = 128, fp16: the V fragments are read before the first softmax, so that the next V tile is requested
    // earlier (B*H = 1 N = 17536 dense block-causal 206 -> 184 us; with bf16 inputs the same order is 5-10 %
    // slower, and at D = 64 the registers are not there)
    constexpr bool EARLY_V = D == 128 && DT == 0;
    uintx4 kfr[2][KS], vfr[4][DB];
    uintx4 pf[4][2];  // P^T operand fragments: [16-key slice][qb]
    auto scores = [&](int qb, floatx16& s0, floatx16& s1) {   // S^T[.][qb] = K Q[qb]^T (- m_i when FOLD)
#pragma unroll
      for (int i = 0; i < 16; ++i) { s0[i] = 0.f; s1[i] = 0.f; }
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        s0 = mfma_qk<BF16>(kfr[0][s], qf[qb][s], s0);
        s1 = mfma_qk<BF16>(kfr[1][s], qf[qb][s], s1);
      }
    };
    // FOLD: "- m_i" through the extra slice, only while some lane of the wavefront has moved its reference
    auto mslice = [&](int qb, floatx16& s0, floatx16& s1) {
      if constexpr (FOLD) {
        if (any_m) {
          s0 = mfma_qk<BF16>(ones_frag, mfrag[qb], s0);
          s1 = mfma_qk<BF16>(ones_frag, mfrag[qb], s1);
        }
      }
    };
    auto read_v = [&]() {
#pragma unroll
      for (int ts = 0; ts < 4; ++ts)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          uintx4 a;
#pragma unroll
          for (int jh = 0; jh < 2; ++jh) {
            const int key = 16 * ts + 8 * jh + vkey0, col = 32 * db + vcol0;
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
    auto second = [&](int qb) {        // O^T[.][qb] += V^T P^T[qb]
#pragma unroll
      for (int ts = 0; ts < 4; ++ts)
#pragma unroll
        for (int db = 0; db < DB; ++db)
          oacc[db][qb] = mfma_qk<PB>(vfr[ts][db], pf[ts][qb], oacc[db][qb]);
    };
    // Softmax numerators, one query per lane.  Fast path: P = exp2(score - m_i) with the
    // reference m_i left alone; the row sum of the fp16-rounded P (what the second product
    // consumes) is accumulated with dot2.  If a lane's sum grows by 2^14 or more (or is not
    // finite), some P left the safe fp16 range: recentre() moves m_i to the tile's row maximum
    // and the numerators are redone from the scores, which are still live.
    auto settle = [&](int qb, floatx16& s0, floatx16& s1, float lnew) {
      // (FOLD: the first tile of a row block keeps the reference at 0 when its sums are of moderate size)
      const bool first = FOLD ? fresh && !(lnew >= 0.25f) : fresh;
      if (__any(first || (EW && l_i[qb] == 0.f) || !(lnew - l_i[qb] < 16384.0f))) {
        recentre<DB, FOLD, EW>(s0, s1, oacc, qb, qk_scale, m_i[qb], l_i[qb], mfrag[qb], fresh, g);
        any_m = 1;
        lnew = softmax_tile<FOLD, PB>(s0, s1, qk_scale, m_i[qb], l_i[qb], pf, qb);
      }
      l_i[qb] = lnew;
    };

    floatx16 sa0, sa1, sb0, sb1;
    wait_vm<CPR>();  // K(cur) has landed (V(cur), issued after it, may still be in flight)
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int s = 0; s < KS; ++s) kfr[kb][s] = *reinterpret_cast<const uintx4*>(lds_k + kaddr[kb][s]);
    // EW: the 64 mask bits of this lane's two queries, shifted so that bit 8(i/4) + i%4 (+ 32 for
    // the second key block) is the key of score register i
    unsigned long long mw0 = 0ull, mw1 = 0ull;
    if constexpr (EW) {
      if (partial) { mw0 = lds_bits[ln] >> (4 * g); mw1 = lds_bits[32 + ln] >> (4 * g); }
    }
    lds_wait();      // the K fragments have arrived: the K buffer is free
    mid();
    if (has1) k_copy_all(kg + (int64_t)cbn * 64 * k_rs, tn);
    auto mask_scores = [&](floatx16& s0, floatx16& s1, unsigned long long mw) {
      const unsigned lo = (unsigned)mw, hi = (unsigned)(mw >> 32);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const unsigned bit = 1u << (8 * (i / 4) + (i % 4));
        s0[i] = (lo & bit) ? s0[i] : -INFINITY;
        s1[i] = (hi & bit) ? s1[i] : -INFINITY;
      }
    };
    // [1]
    scores(0, sa0, sa1);
    mslice(0, sa0, sa1);
    if constexpr (EW) { if (partial) mask_scores(sa0, sa1, mw0); }
    __builtin_amdgcn_sched_barrier(0);
    // [2]
    scores(1, sb0, sb1);
    if constexpr (EARLY_V) {
      if (has1) wait_vm<KOPS>(); else wait_vm<0>();  // V(cur) has landed (K(nxt) may be in flight)
      read_v();
    }
    float lnew0 = softmax_tile<FOLD, PB>(sa0, sa1, qk_scale, m_i[0], l_i[0], pf, 0);
    constexpr int NSC = 2 * KS;
#pragma unroll
    for (int it = 0; it < NSC; ++it) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
      __builtin_amdgcn_sched_group_barrier(0x002, 64 / NSC + 1, 0);   // its share of the VALU work
    }
    __builtin_amdgcn_sched_barrier(0);
    mslice(1, sb0, sb1);
    if constexpr (EW) { if (partial) mask_scores(sb0, sb1, mw1); }
    settle(0, sa0, sa1, lnew0);
    if constexpr (!EARLY_V) {
      if (has1) wait_vm<KOPS>(); else wait_vm<0>();  // V(cur) has landed (K(nxt) may be in flight)
      read_v();
    }
    lds_wait();      // the V fragments have arrived: the V buffer is free
    if (copy_v) v_copy_all(vg + (int64_t)cbn * 64 * v_rs);
    // [3]
    second(0);
    float lnew1 = softmax_tile<FOLD, PB>(sb0, sb1, qk_scale, m_i[1], l_i[1], pf, 1);
#pragma unroll
    for (int it = 0; it < 4 * DB; ++it) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 64 / (4 * DB) + 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    settle(1, sb0, sb1, lnew1);
    fresh = false;
    // [4]
    second(1);
    __builtin_amdgcn_sched_barrier(0);
  };

  // Number of entries r in [0, nb] with rp[r] <= x, for two values of x at once.  The row pointers
  // ascend, so this is a search; it is done in two rounds of one load per lane (64 evenly spaced
  // entries, then the entries between two of them) instead of a chain of dependent scalar loads.
  // Also returns the entries around x: s = rp[c - 1] (the last one <= x) and e = rp[c] (c <= nb).
  // (The entries are compared as rp[r] + gap * r, their positions on the axis the ranges are cut on, moved by
  // the head's first tile; gap = 0: plain tile offsets.)
  auto count_le2 = [&](int64_t x0, int64_t x1, int gap, int& c0, int& c1, int& s0, int& e0, int& s1, int& e1) {
    const int32_t* rpg_ = prm.row_ptr + (int64_t)mh * nb;
    const int step = (nb + 64) / 64;
    auto key = [&](int i, int v) { return (int64_t)v + (int64_t)gap * i; };
    if (step >= 64) {     // very long sequences: plain binary searches
      int lo = -1, hi = nb + 1;
      while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (key(mid, rp[mid]) <= x0) lo = mid; else hi = mid; }
      c0 = hi;
      lo = -1; hi = nb + 1;
      while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (key(mid, rp[mid]) <= x1) lo = mid; else hi = mid; }
      c1 = hi;
      s0 = c0 > 0 ? rp[c0 - 1] : 0; e0 = c0 <= nb ? rp[c0] : 0x7fffffff;
      s1 = c1 > 0 ? rp[c1 - 1] : 0; e1 = c1 <= nb ? rp[c1] : 0x7fffffff;
      return;
    }
    const int i1 = lane * step;
    const bool in1 = i1 <= nb;
    const int v1 = in1 ? rpg_[i1] : 0x7fffffff;
    const int a0 = __builtin_popcountll(__ballot(in1 && key(i1, v1) <= x0)), a1 = __builtin_popcountll(__ballot(in1 && key(i1, v1) <= x1));
    const int b0 = (a0 > 0 ? a0 - 1 : 0) * step, b1 = (a1 > 0 ? a1 - 1 : 0) * step;
    const int j0 = b0 + lane, j1 = b1 + lane;
    // (lane `step` holds the next evenly spaced entry, which is > x: it does not count, but may be e)
    const bool in_w0 = lane <= step && j0 <= nb, in_w1 = lane <= step && j1 <= nb;
    const int w0 = in_w0 ? rpg_[j0] : 0x7fffffff;
    const int w1 = in_w1 ? rpg_[j1] : 0x7fffffff;
    const int k0 = a0 > 0 ? __builtin_popcountll(__ballot(in_w0 && key(j0, w0) <= x0)) : 0;
    const int k1 = a1 > 0 ? __builtin_popcountll(__ballot(in_w1 && key(j1, w1) <= x1)) : 0;
    c0 = b0 + k0;
    c1 = b1 + k1;
    s0 = __builtin_amdgcn_readfirstlane(__shfl(w0, k0 > 0 ? k0 - 1 : 0)); e0 = __builtin_amdgcn_readfirstlane(__shfl(w0, k0));
    s1 = __builtin_amdgcn_readfirstlane(__shfl(w1, k1 > 0 ? k1 - 1 : 0)); e1 = __builtin_amdgcn_readfirstlane(__shfl(w1, k1));
  };

  int* ctr = reinterpret_cast<int*>(ml + NW * 2 * 64);
  int* lcols = ctr + 16;
  // The column indices of the range are staged in LDS: a scalar load per tile would put its whole
  // latency in front of the tile's first LDS wait (scalar loads return out of order, so any wait
  // on the shared counter becomes a wait for all of them).
  typedef const unsigned char __attribute__((address_space(4)))* cbyte_ptr_t;
  // entry t of the column list as staged: column block in the low bits, "partly set" in bit 30
  auto flagged_col = [&](int t) {
    int c = cols[t];
    if constexpr (EW) c |= (int)((cbyte_ptr_t)(uintptr_t)prm.tile_partial)[t] << 30;
    return c;
  };
  constexpr int COL_MASK = 0x3fffffff;
  auto stage_cols = [&](int t_lo, int t_hi) {
    for (int i = threadIdx.x; i < t_hi - t_lo && i < C::COLS_CAP; i += NW * 64) {
      int c = prm.col_idx[t_lo + i];
      if constexpr (EW) c |= (int)prm.tile_partial[t_lo + i] << 30;     // EW: "partly set" rides in bit 30
      lcols[i] = c;
    }
  };

  // Whole row blocks [r_lo, r_hi), one wavefront each: handed out through the LDS counter *rctr
  // (set to r_lo + 2 NW beforehand), written directly, nothing to merge.
  void* obase = out_base(prm, b, h);
  auto run_rows = [&](int r_lo, int r_hi, int* rctr, auto&& col_of) {
    // Tickets r_lo, r_lo + 1, ... stand for the row blocks r_hi - 1, r_hi - 2, ...: with block-causal
    // masks the late row blocks are the long ones, and the long ones should not come last.
    int tick = r_lo + w, tick_next = r_lo + NW + w;   // the first two rounds are fixed
    int kdone = -1;                                    // tile whose K and V copies were issued ahead
    while (tick < r_hi) {
      int drawn = 0;
      if (lane == 0) drawn = atomicAdd(rctr, 1);       // the row block after next
      const int row = r_lo + r_hi - 1 - tick, row_next = r_lo + r_hi - 1 - tick_next;
      const int ta = rp[row], tb = rp[row + 1];
      // first tile of the next row block of this wavefront (prefetched under the last tile)
      const int tn = tick_next < r_hi ? rp[row_next] : 0;
      const bool next_has = tick_next < r_hi && rp[row_next + 1] > tn;
      if (ta < tb) {
        int cx = __builtin_amdgcn_readfirstlane(col_of(ta));      // current tile: column block | flag
        if (kdone != ta) {
          k_copy_all(kg + (int64_t)(cx & COL_MASK) * 64 * k_rs, ta);
          v_copy_all(vg + (int64_t)(cx & COL_MASK) * 64 * v_rs);
        }
        reset_acc();
        load_q(row);
        for (int j = ta; j < tb; ++j) {
          const bool last = j + 1 == tb;
          const bool has1 = !last || next_has;
          const int cxn = has1 ? __builtin_amdgcn_readfirstlane(col_of(last ? tn : j + 1)) : 0;
          tile(has1, cxn & COL_MASK, last ? tn : j + 1, has1, (cx >> 30) != 0, [] {});
          cx = cxn;
        }
        kdone = next_has ? tn : -1;
        // normalise and write the row block
        float lsum[2];
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) lsum[qb] = l_i[qb] + __shfl_xor(l_i[qb], 32);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          const float inv = lsum[qb] > 0.f ? 1.0f / lsum[qb] : 0.f;      // no unmasked key at all: O = 0
          const int64_t qrow = (int64_t)(row * 64 + qb * 32 + ln);
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4)
              store_out4<BF16>(obase, qrow * prm.os[2] + 32 * db + 8 * i4 + 4 * g, prm.out_f32,
                               oacc[db][qb][4 * i4] * inv, oacc[db][qb][4 * i4 + 1] * inv,
                               oacc[db][qb][4 * i4 + 2] * inv, oacc[db][qb][4 * i4 + 3] * inv);
          if (prm.lse != nullptr && g == 0)
            prm.lse[((int64_t)bh * prm.N) + qrow] =
                lsum[qb] > 0.f ? (m_i[qb] + __builtin_amdgcn_logf(lsum[qb])) * 0.6931471805599453f : -INFINITY;
        }
      } else {
        // row block without kept tiles: O = 0, lse = -inf
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          const int64_t qrow = (int64_t)(row * 64 + qb * 32 + ln);
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4)
              store_out4<BF16>(obase, qrow * prm.os[2] + 32 * db + 8 * i4 + 4 * g, prm.out_f32, 0.f, 0.f, 0.f, 0.f);
          if (prm.lse != nullptr && g == 0) prm.lse[((int64_t)bh * prm.N) + qrow] = -INFINITY;
        }
      }
      tick = tick_next;
      tick_next = __builtin_amdgcn_readfirstlane(drawn);
    }
  };

  if constexpr (ROWS) {
    // ================= one wavefront per row block =================
    // The workgroup owns the row blocks whose first kept tile lies in its range [g0, g1); they are
    // handed out to the wavefronts through the LDS counter, and a wavefront runs a whole row block
    // alone and writes its result directly: no merge, no partials.
    int r_lo, r_hi;
    {
      // smallest r with rp[r] >= g = number of r with rp[r] <= g - 1 (capped at nb)
      int u0, u1, u2, u3;
      count_le2(g0 - 1, g1 - 1, 0, r_lo, r_hi, u0, u1, u2, u3);
      r_lo = r_lo < nb ? r_lo : nb;
      r_hi = r_hi < nb ? r_hi : nb;
      if (wg >= hs.Peff - 1) r_hi = nb;    // trailing row blocks without kept tiles
      if (wg == 0) r_lo = 0;               // leading ones
    }
    const int t_lo = rp[r_lo];
    stage_cols(t_lo, rp[r_hi]);
    if (threadIdx.x == 0) *ctr = r_lo + 2 * NW;
    __syncthreads();
    auto col_of = [&](int t) { return t - t_lo < C::COLS_CAP ? lcols[t - t_lo] : flagged_col(t); };
    run_rows(r_lo, r_hi, ctr, col_of);
  } else {
    // ================= all wavefronts on one row block at a time =================
    // Tiles of the range are handed out to the wavefronts dynamically (the LDS counter), because
    // the two wavefronts of a SIMD do not progress at the same rate: each wavefront owns a current
    // tile `cur` and has already drawn its next one `nxt`, so that it can prefetch it.  Tiles are
    // drawn in list order, so a wavefront's tiles increase, and `cur >= seg_b` means "nothing left
    // for me in this row block".  kdone / vdone name the tile whose copy into this wavefront's
    // K / V buffer has been issued; no copy is issued across the merge of a row block, which
    // borrows both buffers of every wavefront (one exchange round for the whole accumulator).
    // first row block of the range: largest r with rp[r] <= g0 < rp[r+1]
    // A range boundary within `snap` tiles of an end of the row block it falls in moves to that end
    // (the nearer one): sharing a row block costs a merge, a published part and a pull, several
    // tiles' worth each, and row blocks of up to 2 `snap` tiles are never shared.  Every workgroup
    // applies the same rule with the same distance to both of its boundaries, so the ranges still tile the list.
    int r;
    {
      // the row blocks in which the two ends of the range lie (positions behind a row block's tiles count as
      // its end), then the tiles themselves
      int c0, c1, s0, e0, s1, e1;
      count_le2(x0 + hs.lo, x1 + hs.lo, hs.gap, c0, c1, s0, e0, s1, e1);
      r = c0 - 1;
      g0 = tile_of_pos(hs, x0, r, s0, e0);
      const int n0 = snap_boundary(snap, g0, s0, e0);
      if (n0 >= e0) ++r;
      g0 = n0;
      if (x1 < hs.X) {
        g1 = tile_of_pos(hs, x1, c1 - 1, s1, e1);
        g1 = snap_boundary(snap, g1, s1, e1);
      } else {
        g1 = hs.lo + hs.T;
      }
      if (g0 >= g1) return;
    }
    int kdone = -1, vdone = -1;
    // The copies of this wavefront's first tile are asked for before anything else (its column index by one
    // scalar load), so that they travel while the column list is staged and Q is read.
    if (g0 + w < g1) {
      const int c0 = flagged_col(g0 + w) & COL_MASK;
      k_copy_all(kg + (int64_t)c0 * 64 * k_rs, g0 + w);
      v_copy_all(vg + (int64_t)c0 * 64 * v_rs);
      kdone = vdone = g0 + w;
    }
    stage_cols(g0, g1);
    if (threadIdx.x == 0) { ctr[0] = g0 + 2 * NW; ctr[3] = 0; }
    __syncthreads();
    auto col_of = [&](int t) { return t - g0 < C::COLS_CAP ? lcols[t - g0] : flagged_col(t); };
    int cur = g0 + w, nxt = g0 + NW + w;      // the first two rounds are fixed
    int cb_nxt = nxt < g1 ? __builtin_amdgcn_readfirstlane(col_of(nxt)) : 0;   // column block of tile nxt
    int t = g0;
    const int32_t* rpg = prm.row_ptr + (int64_t)mh * nb;
    while (t < g1) {
      const int row_s = rp[r], row_e = rp[r + 1];
      if (row_e <= t) { ++r; continue; }          // row block without kept tiles in the range
      // A run of short row blocks that lie completely inside the range is not worth a merge per
      // row block: such a run is done one row block per wavefront.  Every wavefront looks at the
      // next 64 row blocks (one per lane) and comes to the same decision.
      if (t == row_s && row_e <= g1 && row_e - row_s <= C::SHORT_ROW) {
        const int idx = r + lane;
        const int rs_i = idx < nb ? rpg[idx] : 0, re_i = idx < nb ? rpg[idx + 1] : 0x7fffffff;
        const bool ok_i = idx < nb && re_i <= g1 && re_i - rs_i <= C::SHORT_ROW;
        const unsigned long long okm = __ballot(ok_i);
        const int cnt = ~okm == 0ull ? 64 : __builtin_ctzll(~okm);        // leading run of short inner row blocks
        const bool in_run = lane < cnt;
        const int bn = __builtin_popcountll(__ballot(in_run && re_i > rs_i));   // ... with kept tiles
        int maxlen = in_run ? re_i - rs_i : 0;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) { const int o = __shfl_xor(maxlen, off); maxlen = o > maxlen ? o : maxlen; }
        maxlen = __builtin_amdgcn_readfirstlane(maxlen);
        // worth it when the run keeps the wavefronts busy, or when its row blocks are short
        // against the cost of a merge (about three tiles per wavefront)
        const bool batch = bn >= NW || (bn == 3) || (bn == 2 && maxlen < 3 * NW) || (bn == 1 && maxlen < NW);
        if (batch) {
          const int r2 = r + cnt, t2 = __builtin_amdgcn_readfirstlane(__shfl(re_i, cnt - 1));
          wait_vm<0>();                 // prefetches of the tile hand-out below are abandoned
          __syncthreads();              // everybody has left the previous run and the previous merge
          if (threadIdx.x == 0) { ctr[2] = r + 2 * NW; ctr[0] = t2 + 2 * NW; }
          __syncthreads();
          run_rows(r, r2, ctr + 2, col_of);
          cur = t2 + w; nxt = t2 + NW + w;
          cb_nxt = nxt < g1 ? __builtin_amdgcn_readfirstlane(col_of(nxt)) : 0;
          kdone = -1; vdone = -1;
          t = t2; r = r2;
          continue;
        }
      }
      const int seg_a = t, seg_b = row_e < g1 ? row_e : g1;
      const bool mine = cur < seg_b;      // this wavefront processes at least one tile of the row block
      reset_acc();
      if (mine) {
        int cx = __builtin_amdgcn_readfirstlane(col_of(cur));     // current tile: column block | flag
        if (kdone != cur) { k_copy_all(kg + (int64_t)(cx & COL_MASK) * 64 * k_rs, cur); kdone = cur; }
        if (vdone != cur) { v_copy_all(vg + (int64_t)(cx & COL_MASK) * 64 * v_rs); vdone = cur; }
        load_q(r);
        while (cur < seg_b) {
          // draw the tile after next; the value is picked up inside the tile
          int drawn = 0;
          if (lane == 0) drawn = atomicAdd(ctr, 1);
          // the next tile is only prefetched inside the row block: the merge at its end borrows both buffers
          const bool has1 = nxt < seg_b, copy_v = has1;
          int nn = 0, cb_nn_v = 0;
          tile(has1, cb_nxt & COL_MASK, nxt, copy_v, (cx >> 30) != 0, [&] {
            // (deterministic: every wavefront takes every NW-th tile, whatever its pace)
            nn = prm.deterministic ? nxt + NW : __builtin_amdgcn_readfirstlane(drawn);
            cb_nn_v = nn < g1 ? col_of(nn) : 0;     // looked up now, needed at the end of the tile
          });
          if (has1) kdone = nxt;
          if (copy_v) vdone = nxt;
          cur = nxt;
          cx = cb_nxt;
          nxt = nn;
          cb_nxt = __builtin_amdgcn_readfirstlane(cb_nn_v);
        }  // tiles of this wavefront
      }
      // ---- merge the wavefronts' results of this row block through LDS ----
      // Each wavefront publishes (m, l) per query and, round by round, R accumulator registers in
      // its own V buffer ([register][lane] floats); in every round each wavefront reduces QPW
      // groups of 4 registers (4 consecutive head-dimension values of one query per lane) over all
      // contributing wavefronts and writes them out.
      {
        // (a wavefront without tiles in the range's first row block may still have its first tile's copies in
        // flight: the merge borrows the tile buffers, so they are waited for and asked for again afterwards)
        if (!mine) { wait_vm<0>(); kdone = -1; vdone = -1; }
        float lsum[2];
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) lsum[qb] = l_i[qb] + __shfl_xor(l_i[qb], 32);
        if (g == 0) {
#pragma unroll
          for (int qb = 0; qb < 2; ++qb) {
            const bool mass = mine && lsum[qb] > 0.f;
            ml[(w * 2 + 0) * 64 + qb * 32 + ln] = mass ? m_i[qb] : -INFINITY;
            ml[(w * 2 + 1) * 64 + qb * 32 + ln] = mass ? lsum[qb] : 0.f;
          }
        }
        // A row block cut by range boundaries has one part per workgroup that holds tiles of it.  Every
        // such workgroup publishes its part and then counts itself in; the one that finds all the
        // others counted merges the parts and writes the row block.  Nobody waits for anybody, so
        // the result does not depend on which workgroups are resident at the same time.
        const bool has_head = seg_a == row_s, has_tail = seg_b == row_e;
        const bool full = has_head && has_tail;
        float wgt[NW][2];   // weight of wavefront p's partial for this lane's query of block qb
        float M[2], L[2];
        float keep[C::ROUNDS][C::QPW][4];   // this wavefront's share of the workgroup's part
        // parts travel 16 bytes per lane and access at D = 64 (N = 17536, one head: dense 101.6 -> 101.0 us, keep 0.25
        // 41.8 -> 41.1, keep 0.05 20.6 -> 20.0); at D = 128 that is faster for long ranges (keep 0.5 241 -> 233 us) and
        // slower for short ones (keep 0.07 79 -> 82 us), and choosing by regime at run time gains nothing: 4 bytes there
        constexpr bool WIDE_PARTS = D == 64;
        // A zero the compiler cannot see through (ctr[3] stays 0): the per-lane addresses into the
        // workspace do not change from row block to row block and would otherwise be computed
        // once, up front, and occupy registers throughout the tile loops.
        typedef volatile int __attribute__((address_space(3)))* lds_vint_ptr_t;
        const int zero = *(lds_vint_ptr_t)(lds_ptr_t)(ctr + 3);
        // two slots per workgroup: a range can end inside one row block (that part goes to slot 1: it
        // holds the row block's first tiles) after having begun inside another (slot 0)
        auto slot_of = [&](int p, bool head) {
          return prm.ws + (((int64_t)bh * prm.W + p) * 2 + (head ? 1 : 0)) * partial_floats(D) + zero;
        };
        float* slot = slot_of(wg, has_head);
        // A part's holder looks at the arrival counter now: the value is only the first guess of the
        // compare-and-swap below, and its round trip runs beside the merge instead of behind it.
        unsigned long long* arrivals = prm.flags + (int64_t)bh * nb + r;
        unsigned long long seen = 0;
        if (!full && threadIdx.x == 0) seen = __hip_atomic_load(arrivals, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int rd = 0; rd < C::ROUNDS; ++rd) {
          {
            // every wavefront writes (one without tiles of this row block holds zeros), 4 bytes per
            // lane and instruction: wider LDS writes are much slower per byte on this hardware
            float* own = reinterpret_cast<float*>(lds_k);
#pragma unroll
            for (int e = 0; e < C::R; ++e) {
              const int idx = rd * C::R + e;
              own[e * 64 + lane] = oacc[idx / 32][(idx / 16) & 1][idx & 15];
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
              const float* src = reinterpret_cast<const float*>(lds + pw * C::WAVE_LDS);
#pragma unroll
              for (int e = 0; e < 4; ++e) x[e] += wgt[pw][qb] * src[(4 * quad + e) * 64 + lane];
            }
            if (full) {
              const float inv = L[qb] > 0.f ? 1.0f / L[qb] : 0.f;
              const int64_t qrow = (int64_t)(r * 64 + qb * 32 + ln);
              store_out4<BF16>(obase, qrow * prm.os[2] + 32 * db + 8 * i4 + 4 * g, prm.out_f32, x[0] * inv, x[1] * inv,
                               x[2] * inv, x[3] * inv);
            } else {
              // (WIDE_PARTS: 16 bytes per lane and access, the part laid out [quad][lane][4])
              if constexpr (WIDE_PARTS) {
                coherent_store4(slot + idx0 * 64 + lane * 4, x[0], x[1], x[2], x[3]);
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) coherent_store(slot + (idx0 + e) * 64 + lane, x[e]);
              }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) keep[rd][tq][e] = x[e];
          }
          __syncthreads();
        }
        if (full) {
          if (w == 0 && g == 0 && prm.lse != nullptr) {
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
              prm.lse[((int64_t)bh * prm.N) + (int64_t)(r * 64 + qb * 32 + ln)] =
                  L[qb] > 0.f ? (M[qb] + __builtin_amdgcn_logf(L[qb])) * 0.6931471805599453f : -INFINITY;
          }
        } else {
          if (w == 0 && g == 0) {
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
              coherent_store(slot + 64 * D + qb * 32 + ln, M[qb]);
              coherent_store(slot + 64 * D + 64 + qb * 32 + ln, L[qb]);
            }
          }
          // The workgroups pf .. pl hold the parts of this row block: pf is the one before the first range
          // boundary that stays inside the row block (boundaries close to an end move there), pl the one
          // after the last.  Every holder computes the same two numbers.
          const int64_t xrow = row_pos(hs, r, row_s);
          int pl_ = split_of_pos(hs, xrow + (row_e - 1 - row_s)), pf_ = split_of_pos(hs, xrow);
          while (pl_ > pf_ && snap_boundary(snap, tile_of_pos(hs, split_pos(hs, pl_), r, row_s, row_e), row_s, row_e) >= row_e) --pl_;
          while (pf_ < pl_ && snap_boundary(snap, tile_of_pos(hs, split_pos(hs, pf_ + 1), r, row_s, row_e), row_s, row_e) <= row_s) ++pf_;
          const int nparts = pl_ - pf_ + 1;
          // The part is counted in once every wavefront's stores have been acknowledged (vmcnt 0, then the
          // barrier).  Every access to a part, stores here and loads below, is itself an access at device
          // scope: it is served by the memory all compute units share, never by a cache that only
          // some of them see.  The counter update is therefore relaxed: release / acquire order on it
          // would add a write-back and an invalidation of this die's whole L2, measured at 9 us per
          // launch (keep 0.1, N = 17536: 31 -> 41 us), to order accesses that are already ordered.
          // The counter holds (launch mark << 16 | parts counted); stale contents carry another mark.
          wait_vm<0>();
          __syncthreads();
          if (threadIdx.x == 0) {
            unsigned long long old = seen;
            for (;;) {     // (ends: the counter only changes when another part is counted, at most nparts times)
              const unsigned long long want = (old >> 16) == prm.epoch ? old + 1 : ((prm.epoch << 16) | 1ull);
              if (__hip_atomic_compare_exchange_strong(arrivals, &old, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT)) {
                ctr[4] = (int)(want & 0xffffull);
                break;
              }
            }
          }
          __syncthreads();
          const int counted = __builtin_amdgcn_readfirstlane(*(lds_vint_ptr_t)(lds_ptr_t)(ctr + 4));
          if (counted == nparts) {
            // last one in: every part is in memory.  They are summed in the order of the ranges, whoever
            // does it, so the result does not depend on the order of arrival.
            float Ms[2] = {-INFINITY, -INFINITY}, Ls[2] = {0.f, 0.f}, acc[C::ROUNDS][C::QPW][4];
#pragma unroll
            for (int rd = 0; rd < C::ROUNDS; ++rd)
#pragma unroll
              for (int tq = 0; tq < C::QPW; ++tq)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[rd][tq][e] = 0.f;
            for (int p = pf_; p <= pl_; ++p) {
              float mp[2], lp[2], dat[C::ROUNDS][C::QPW][4];
              if (p == wg) {
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) { mp[qb] = M[qb]; lp[qb] = L[qb]; }
#pragma unroll
                for (int rd = 0; rd < C::ROUNDS; ++rd)
#pragma unroll
                  for (int tq = 0; tq < C::QPW; ++tq)
#pragma unroll
                    for (int e = 0; e < 4; ++e) dat[rd][tq][e] = keep[rd][tq][e];
              } else {
                const float* sp = slot_of(p, p == pf_);
                // all loads of the part are issued before the first one is waited for (a round trip
                // to the point of coherence costs about a microsecond)
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
                  mp[qb] = coherent_load(sp + 64 * D + qb * 32 + ln);
                  lp[qb] = coherent_load(sp + 64 * D + 64 + qb * 32 + ln);
                }
                if constexpr (WIDE_PARTS) {
                  static_assert(!WIDE_PARTS || (C::ROUNDS == 1 && C::QPW == 4), "four 16-byte loads per lane and part");
                  floatx4 ld[4];
                  coherent_load4x4(sp + 4 * (w * C::QPW) * 64 + lane * 4, ld[0], ld[1], ld[2], ld[3]);   // ([quad][lane][4]: a quad is 1 KB)
#pragma unroll
                  for (int rd = 0; rd < C::ROUNDS; ++rd)
#pragma unroll
                    for (int tq = 0; tq < C::QPW; ++tq)
#pragma unroll
                      for (int e = 0; e < 4; ++e) dat[rd][tq][e] = ld[rd * C::QPW + tq][e];
                } else {
#pragma unroll
                  for (int rd = 0; rd < C::ROUNDS; ++rd)
#pragma unroll
                    for (int tq = 0; tq < C::QPW; ++tq)
#pragma unroll
                      for (int e = 0; e < 4; ++e)
                        dat[rd][tq][e] = coherent_load(sp + (rd * C::R + 4 * (w * C::QPW + tq) + e) * 64 + lane);
                  __builtin_amdgcn_sched_barrier(0);
                }
              }
              float sc_own[2], sc_p[2];
#pragma unroll
              for (int qb = 0; qb < 2; ++qb) {
                const float mn = fmaxf(Ms[qb], mp[qb]);     // a side without mass has maximum -inf and weight 0
                sc_own[qb] = Ms[qb] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(Ms[qb] - mn);
                sc_p[qb] = mp[qb] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mp[qb] - mn);
                Ls[qb] = Ls[qb] * sc_own[qb] + lp[qb] * sc_p[qb];
                Ms[qb] = mn;
              }
#pragma unroll
              for (int rd = 0; rd < C::ROUNDS; ++rd)
#pragma unroll
                for (int tq = 0; tq < C::QPW; ++tq) {
                  const int qb = ((rd * C::R + 4 * (w * C::QPW + tq)) / 16) & 1;
#pragma unroll
                  for (int e = 0; e < 4; ++e) acc[rd][tq][e] = acc[rd][tq][e] * sc_own[qb] + sc_p[qb] * dat[rd][tq][e];
                }
            }
#pragma unroll
            for (int rd = 0; rd < C::ROUNDS; ++rd)
#pragma unroll
              for (int tq = 0; tq < C::QPW; ++tq) {
                const int idx0 = rd * C::R + 4 * (w * C::QPW + tq);
                const int db = idx0 / 32, qb = (idx0 / 16) & 1, i4 = (idx0 & 15) / 4;
                const float inv = Ls[qb] > 0.f ? 1.0f / Ls[qb] : 0.f;
                const int64_t qrow = (int64_t)(r * 64 + qb * 32 + ln);
                store_out4<BF16>(obase, qrow * prm.os[2] + 32 * db + 8 * i4 + 4 * g, prm.out_f32,
                                 acc[rd][tq][0] * inv, acc[rd][tq][1] * inv, acc[rd][tq][2] * inv, acc[rd][tq][3] * inv);
              }
            if (w == 0 && g == 0 && prm.lse != nullptr) {
#pragma unroll
              for (int qb = 0; qb < 2; ++qb)
                prm.lse[((int64_t)bh * prm.N) + (int64_t)(r * 64 + qb * 32 + ln)] =
                    Ls[qb] > 0.f ? (Ms[qb] + __builtin_amdgcn_logf(Ls[qb])) * 0.6931471805599453f : -INFINITY;
            }
            // back to zero, so that a replay of this launch (same mark) starts from a clean counter
            if (threadIdx.x == 0) __hip_atomic_store(arrivals, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      }
      t = seg_b;
      ++r;
    }
  }
}

// A 48-bit number that differs from launch to launch (and, through its start value, from process
// to process); never zero.
unsigned long long next_epoch() {
  static std::atomic<unsigned long long> counter{
      (unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count() * 0x9E3779B97F4A7C15ull};
  unsigned long long e;
  do { e = counter.fetch_add(1) & 0xffffffffffffull; } while (e == 0);
  return e;
}

// Process-wide switch: results that do not depend on the pace of the wavefronts (bsattn_set_deterministic).
static std::atomic<int> deterministic_mode{0};
int set_deterministic(int on) { return deterministic_mode.exchange(on != 0 ? 1 : 0); }
int get_deterministic() { return deterministic_mode.load(); }

int compute_units() {
  static int cached[64] = {0};   // per device; the value never changes, so a race only repeats the query
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) != hipSuccess) return cus;
  if (dev >= 0 && dev < 64 && cached[dev] > 0) return cached[dev];
  int v = 0;
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  if (dev >= 0 && dev < 64) cached[dev] = cus;
  return cus;
}

static int groups_per_head(int B, int H, int nb, int D) {
  const int cus = compute_units();
  const int per_cu = D == 64 ? FwdCfg<64>::WG_PER_CU : FwdCfg<128>::WG_PER_CU;
  int64_t W = (int64_t)cus * per_cu / ((int64_t)B * H);   // as many workgroups as are resident at once
  const int64_t cap = (int64_t)nb * nb;
  if (W > cap) W = cap;
  if (W < 1) W = 1;
  return (int)W;
}

// workspace: partial slots [B*H][W][2][partial_floats] (fp32), then the arrival counters [B*H][nb] (64 bit)
static size_t slots_bytes(int B, int H, int W, int D) {
  return (size_t)B * H * W * 2 * partial_floats(D) * sizeof(float);
}

// Pair kernel: workgroups per row block.  One when the launch has enough row blocks to fill the GPU twice
// over; otherwise the row lists are shared (up to 8 ways, a share of a dense list keeping at least 8 tiles).
static int pair_split(int B, int H, int nb, int D) {
  const int64_t row_blocks = (int64_t)B * H * nb;
  const int64_t want = (int64_t)compute_units() * (D == 128 ? 4 : 2) * 2;
  if (row_blocks >= want) return 1;
  int64_t s = (want + row_blocks - 1) / row_blocks;
  const int cap = nb / 8 > 1 ? nb / 8 : 1;
  if (s > cap) s = cap;
  return (int)(s > 8 ? 8 : s);
}

static size_t pair_parts_bytes(int B, int H, int N, int D, int split) {
  return split > 1 ? (size_t)split * B * H * N * (D + 2) * sizeof(float) : 0;
}

size_t coop_workspace_bytes(int B, int H, int N, int D) {
  if (D == 256) return 256 + pair_parts_bytes(B, H, N, D, pair_split(B, H, N / 64, D));   // the pair kernel only
  const int nb = N / 64;
  const int W = groups_per_head(B, H, nb, D);
  return slots_bytes(B, H, W, D) + (size_t)B * H * nb * sizeof(unsigned long long);
}

// one size for bsattn_fwd and bsattn_fwd_elementwise
size_t fwd_workspace_bytes(int B, int H, int N, int D) { return coop_workspace_bytes(B, H, N, D); }

void launch_fwd_pair(const FwdParams& prm, int D, int dt, bool elementwise, hipStream_t st);   // attn_fwd_pair.hip
// D = 128 with enough row blocks in the launch to fill the chip goes to the kernel that gives each
// row block to one wavefront pair (two wavefronts per SIMD, no merges between workgroups).  With
// fewer row blocks its critical path is the longest row, which the host cannot see (the lists
// stay on the device): from two row blocks per compute unit on it won in every measured case,
// from one on only when rows are short (at most 32 tiles).
static bool use_pair_kernel(int64_t row_blocks, int nb) {
  const int64_t cus = compute_units();
  return row_blocks >= 2 * cus || (row_blocks >= cus && nb <= 32);
}

// With few row blocks per workgroup all wavefronts of a workgroup share one row block at a time
// (K and V tiles are spread over them and the results merged); with many (>= 8 per workgroup) each
// wavefront takes whole row blocks, which needs no merge and no second kernel.
static bool rows_mode(const FwdParams& prm) { return prm.nb >= 8 * prm.W; }

template <int D, int DT, bool EW, bool CONTIG>
static void launch_fwd_c(const FwdParams& prm, int BH, hipStream_t st) {
  using C = FwdCfg<D>;
  static std::atomic<unsigned long long> configured{0};   // raising the dynamic LDS limit is idempotent
  once_per_device(configured, [] {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&fwd_kernel<D, DT, false, EW, CONTIG>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&fwd_kernel<D, DT, true, EW, CONTIG>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
  });
  if (rows_mode(prm)) {
    hipLaunchKernelGGL((fwd_kernel<D, DT, true, EW, CONTIG>), dim3(prm.W * BH), dim3(C::NW * 64), C::LDS_BYTES, st, prm);
  } else {
    hipLaunchKernelGGL((fwd_kernel<D, DT, false, EW, CONTIG>), dim3(prm.W * BH), dim3(C::NW * 64), C::LDS_BYTES, st, prm);
  }
}

// The copies with immediate offsets are compiled where they were measured faster: D = 64 (2-4 %) and
// D = 128 with bf16 inputs (4-8 %; with fp16 inputs 1-3 % slower).
template <int D, int DT, bool EW>
static void launch_fwd_t(const FwdParams& prm, int BH, hipStream_t st) {
  constexpr bool HAS_CONTIG = D == 64 || DT != 0;
  if (HAS_CONTIG && prm.ks[2] == D && prm.vs[2] == D) launch_fwd_c<D, DT, EW, HAS_CONTIG>(prm, BH, st);
  else launch_fwd_c<D, DT, EW, false>(prm, BH, st);
}

// ---- forward without any allocation by anybody: the scratch memory is part of the library ----
// A file-scope device array stands in for the workspace argument of launch_fwd.  In host code its name
// is only a handle: the address the kernels may use is asked for once per device (each device holds
// its own copy of the array at its own address).
static __device__ __align__(256) unsigned char scratch[BSATTN_STATIC_SCRATCH_BYTES];

int static_scratch(void** ptr) {
  static std::atomic<void*> per_device[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return BSATTN_ERR_LAUNCH;
  void* p = per_device[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    // (two threads may both ask: they get the same answer)
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return BSATTN_ERR_LAUNCH;
    per_device[dev].store(p, std::memory_order_release);
  }
  *ptr = p;
  return BSATTN_OK;
}

// The range permutation of fwd_kernel (range_perm.h) depends on (nb, W, F, heads) only: kept in a small cache.
static bool range_permutation(int nb, int W, int F, int BH, unsigned short* out, unsigned short* out_causal) {
  static std::mutex mu;
  static std::map<std::array<int, 4>, std::array<unsigned short, 2 * RANGE_PERM_MAX>> cache;
  const std::array<int, 4> key = {nb, W, F, BH};
  std::lock_guard<std::mutex> lock(mu);
  auto it = cache.find(key);
  if (it == cache.end()) {
    std::array<unsigned short, 2 * RANGE_PERM_MAX> t{};
    if (!make_range_permutation(nb, W, F, BH, WEIGHT_FAST, WEIGHT_SLOW, false, t.data()) ||
        !make_range_permutation(nb, W, F, BH, WEIGHT_FAST, WEIGHT_SLOW, true, t.data() + RANGE_PERM_MAX)) return false;
    if (cache.size() >= 64) cache.clear();
    it = cache.emplace(key, t).first;
  }
  for (int i = 0; i < W; ++i) { out[i] = it->second[i]; out_causal[i] = it->second[RANGE_PERM_MAX + i]; }
  return true;
}

int launch_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
               const int32_t* row_ptr, const int32_t* col_idx, const uint8_t* tile_partial,
               const uint64_t* tile_bits, const AttnShape& s, void* ws, hipStream_t st) {
  FwdParams prm;
  prm.q = q; prm.k = k; prm.v = v; prm.o = o; prm.lse = lse;
  prm.row_ptr = row_ptr; prm.col_idx = col_idx; prm.ws = (float*)ws;
  prm.tile_partial = tile_partial; prm.tile_bits = (const unsigned long long*)tile_bits;
  prm.B = s.B; prm.H = s.H; prm.N = s.N; prm.nb = s.N / 64; prm.Bm = s.Bm; prm.Hm = s.Hm;
  prm.W = groups_per_head(s.B, s.H, prm.nb, s.D);
  // with two workgroups per compute unit the first-comers are faster: tell the kernel which they are
  prm.first_ids = (s.D == 64 ? FwdCfg<64>::WG_PER_CU : FwdCfg<128>::WG_PER_CU) > 1 ? compute_units() : 0;
  prm.flags = (unsigned long long*)((char*)ws + slots_bytes(s.B, s.H, prm.W, s.D));
  prm.epoch = next_epoch();
  prm.deterministic = get_deterministic();
  {
    const int BHl = s.B * s.H;
    const int F = prm.first_ids > 0 && prm.first_ids % BHl == 0 ? (prm.first_ids / BHl < prm.W ? prm.first_ids / BHl : prm.W) : 0;
    const bool ok = (prm.first_ids == 0 || prm.first_ids % BHl == 0) && range_permutation(prm.nb, prm.W, F, BHl, prm.perm, prm.perm_causal);
    prm.perm_n = ok ? prm.W : 0;
    prm.perm_fast = F;
    prm.perm_min_tiles = (int)((int64_t)prm.nb * prm.nb * 3 / 4);
  }
  prm.out_f32 = s.out_dtype == BSATTN_F32;
  prm.qk_scale = s.sm_scale * 1.4426950408889634f;
  for (int i = 0; i < 3; ++i) { prm.qs[i] = s.qs[i]; prm.ks[i] = s.ks[i]; prm.vs[i] = s.vs[i]; prm.os[i] = s.os[i]; }
  const bool bf = s.dtype == BSATTN_BF16;
  const int BH = s.B * s.H;
  prm.split = 1;
  if (s.D == 256 || (s.D == 128 && use_pair_kernel((int64_t)BH * prm.nb, prm.nb))) {   // (D = 256 has no other kernel)
    // D = 256 launches with few row blocks share the row lists between workgroups; at D = 128 the
    // cooperative kernel below takes those launches (sharing was measured: faster on dense masks with 2-3
    // heads, 25-30 % slower on sparse ones)
    if (s.D == 256) prm.split = pair_split(s.B, s.H, prm.nb, s.D);
    prm.part_o = (float*)ws + 64;
    prm.part_ml = prm.part_o + (size_t)prm.split * BH * s.N * s.D;
    launch_fwd_pair(prm, s.D, !bf ? 0 : (prm.out_f32 ? 1 : 2), tile_bits != nullptr, st);
    return launch_status();
  }
  // bf16 with a bf16-typed result: P is rounded to bf16 as well (the reference rounds P to the type of
  // V, fa2_fwd.py:189) and V is used as it is; an fp32 result keeps P in fp16
  const int dt = !bf ? 0 : (prm.out_f32 ? 1 : 2);
  if (tile_bits == nullptr) {
    if (s.D == 64) { if (dt == 0) launch_fwd_t<64, 0, false>(prm, BH, st); else if (dt == 1) launch_fwd_t<64, 1, false>(prm, BH, st); else launch_fwd_t<64, 2, false>(prm, BH, st); }
    else { if (dt == 0) launch_fwd_t<128, 0, false>(prm, BH, st); else if (dt == 1) launch_fwd_t<128, 1, false>(prm, BH, st); else launch_fwd_t<128, 2, false>(prm, BH, st); }
  } else {   // elementwise mask
    if (s.D == 64) { if (dt == 0) launch_fwd_t<64, 0, true>(prm, BH, st); else if (dt == 1) launch_fwd_t<64, 1, true>(prm, BH, st); else launch_fwd_t<64, 2, true>(prm, BH, st); }
    else { if (dt == 0) launch_fwd_t<128, 0, true>(prm, BH, st); else if (dt == 1) launch_fwd_t<128, 1, true>(prm, BH, st); else launch_fwd_t<128, 2, true>(prm, BH, st); }
  }
  return launch_status();
}

}  // namespace bsattn
