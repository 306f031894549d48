// Block-sparse FlashAttention-2 forward for gfx950, head dimension 64: the kernel for masks whose
// neighbouring row blocks keep (nearly) the same column blocks: dense, block-causal, banded, frame-wise.
// Correct for every block mask; fast when the four row lists of a quad agree.
//
// Two things keep the matrix cores of a SIMD fed here.
//  (1) K and V tiles are shared.  A wavefront group is four wavefronts, one per SIMD, that own the
//      four row blocks of a quad (64 queries each) and walk the union of the quad's four column
//      lists together: every K and V tile is copied into LDS once per group (each wavefront issues
//      a quarter of the copy) and read by all four.  A wavefront whose row block does not keep the
//      current column block sits the tile out.
//  (2) Matrix and vector work alternate between two groups.  A workgroup holds two groups (two
//      wavefronts per SIMD).  Per tile a wavefront has a matrix phase (second product of the previous
//      tile, first product of this one: 36 MFMAs, no vector work) and a vector phase (the softmax
//      numerators: exponentials, conversions, row sums, no MFMA).  The groups run one phase apart,
//      separated by workgroup barriers, so on every SIMD one wavefront is in its matrix phase while
//      the other is in its vector phase.
//
// The union lists come from the mask preprocessing (quad_union_kernel, mask_index.hip): per quad the
// column blocks any of its rows keeps, each with the membership of the four rows.
// Work split (fwd_quad_split.h): the quads of the launch lie on a weight axis (a quad weighs the size of
// its union list) that is cut into one range per group.  A quad cut by range boundaries is finished by whichever group arrives last: every group
// writes its unnormalised part (accumulator, reference exponent, row sum per row block) to the
// workspace with device-scope stores, waits for their acknowledgement and counts itself in on the row
// block's counter; the one that completes the count reads all parts in part order and writes the row
// block.  Nobody waits for anybody, so the kernel does not depend on which workgroups are resident.
//
// The tile arithmetic is that of fwd_kernel (attn_fwd.hip): S^T = K Q^T with one query per lane,
// recurrence of the reference kernel fa2_custom_mask/fa2_fwd.py:146-196.
#include <type_traits>
#include "common.h"
#include "fwd_quad_split.h"
#include "fwd_split.h"
#include "fwd_tile.h"
#include "kernel_util.h"

namespace bsattn {

struct QuadCfg {
  static constexpr int D = 64;
  static constexpr int TILE_BYTES = 64 * 2 * D;           // 8 KB
  static constexpr int GROUP_TILES = 5 * TILE_BYTES;      // K0 K1 K2 V0 V1 of one group
  static constexpr int NB_CAP = 2048;                     // column blocks a quad's list may hold
  static constexpr int LIST_BYTES = NB_CAP * 4;
  static constexpr int CUM_CAP = 4096;                    // quads per period of the weight axis
  static constexpr int OFF_LISTS = 2 * GROUP_TILES;                       // [2 groups][3][NB_CAP] ints
  static constexpr int OFF_CUM = OFF_LISTS + 2 * 3 * LIST_BYTES;          // [CUM_CAP + 1] ints
  static constexpr int OFF_DESC = OFF_CUM + (CUM_CAP + 64) * 4;           // [2 groups][3][8] ints
  static constexpr int LDS_BYTES = OFF_DESC + 2 * 3 * 8 * 4;
};

// 16 bytes per lane to / from memory that other workgroups read / wrote during this launch: device
// scope, served at the point of coherence.  The loads are not tracked by the compiler: wait with
// coherent_wait() on the loaded values before using them.
__device__ __forceinline__ void coherent_store4(float* p, floatx4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1" :: "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ floatx4 coherent_load4(const float* p) {
  floatx4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
  return v;
}

// inclusive sum over the lanes of a wavefront
__device__ __forceinline__ int wave_inclusive_sum(int v, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int o = __shfl_up(v, off);
    if (lane >= off) v += o;
  }
  return v;
}

// Measurement build only (-DQUAD_TIMELINE, never the library's): every wavefront group writes the 100 MHz
// wall clock at four points (entry, first round, last round done, row blocks finished) to a buffer whose
// address the launcher takes from the environment variable BSATTN_QUAD_TIMELINE.
#ifdef QUAD_TIMELINE
#define QUAD_WALL(i) do { if (prm.part_o != nullptr && (threadIdx.x & 255) == 0) \
    reinterpret_cast<long long*>(prm.part_o)[(blockIdx.x * 2 + (threadIdx.x >> 8)) * 4 + (i)] = __builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define QUAD_WALL(i) do {} while (0)
#endif

template <int DT, bool CONTIG>
__global__ __launch_bounds__(512, 1)
void fwd_quad_kernel(const FwdParams prm) {
  constexpr int D = 64;
  constexpr bool BF16 = DT != 0, PB = DT == 2;     // DT 1: bf16 inputs, P rounded to fp16 (the transposed V copy is fp16 then)
  constexpr bool FOLD = !BF16;
  constexpr int KS = D / 16, DB = D / 32, CPR = D / 8, ROWB = 2 * D;
  using C = QuadCfg;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

  const int lane = threadIdx.x & 63;
  QUAD_WALL(0);
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = w >> 2, r = w & 3;     // wavefronts r and r + 4 share a SIMD
  const int ln = lane & 31, g = lane >> 5;
  const int nb = prm.nb, nq = (nb + 3) >> 2, BH = prm.B * prm.H;
  const bool shared_mask = prm.Bm == 1 && prm.Hm == 1;

  // ---- row blocks without kept tiles: O = 0, lse = -inf, dealt round-robin over the workgroups ----
  for (int rb = blockIdx.x; rb < BH * nb; rb += gridDim.x) {
    const int bh = rb / nb, row = rb - bh * nb;
    const int32_t* rpm = prm.row_ptr + (int64_t)(shared_mask ? 0 : bh) * nb;
    if (rpm[row + 1] > rpm[row]) continue;
    const int b = bh / prm.H, h = bh - b * prm.H;
    void* ob = out_base(prm, b, h);
    for (int i = threadIdx.x; i < 64 * (D / 4); i += 512) {
      const int64_t qrow = (int64_t)row * 64 + i / (D / 4);
      store_out4<BF16>(ob, qrow * prm.os[2] + 4 * (i % (D / 4)), prm.out_f32, 0.f, 0.f, 0.f, 0.f);
    }
    if (prm.lse != nullptr && threadIdx.x < 64) prm.lse[(int64_t)bh * prm.N + (int64_t)row * 64 + threadIdx.x] = -INFINITY;
  }

  // ---- the weight axis: the prefix sums of the union sizes of one period, copied into LDS ----
  // (every wavefront writes the same values; each reads only after its own writes)
  int32_t* cum = reinterpret_cast<int32_t*>(lds + C::OFF_CUM);
  const int period_quads = shared_mask ? nq : BH * nq;
  for (int i = lane; i <= period_quads; i += 64) cum[i] = prm.quad_ptr[i];
  const int period_weight = __builtin_amdgcn_readfirstlane(cum[period_quads]);
  if (period_weight == 0) return;     // nothing kept anywhere
  // the axis as the split functions see it: reads of cum[] are wavefront-uniform LDS reads, the search
  // compares 64 entries at a time
  struct UniformCum {
    const int32_t* p;
    __device__ __forceinline__ int operator[](int i) const { return __builtin_amdgcn_readfirstlane(p[i]); }
  };
  struct Axis {
    UniformCum cum; int period_quads, period_weight, reps, slots, lane;
    __device__ __forceinline__ int64_t total() const { return (int64_t)period_weight * reps; }
    __device__ __forceinline__ int find(int xr) const {     // entries 1 .. period_quads that are <= xr
      int n = 0;
      for (int base = 1; base <= period_quads; base += 64) {
        const int i = base + lane;
        n += __builtin_popcountll(__ballot(i <= period_quads && cum.p[i] <= xr));
      }
      return n;
    }
  } axis{UniformCum{cum}, period_quads, period_weight, shared_mask ? BH : 1, 1, lane};
  axis.slots = quad_slots(axis.total(), 2 * (int)gridDim.x);
  const int slot = 2 * blockIdx.x + grp;
  if (slot >= axis.slots) return;
  const int64_t x_begin = quad_cut(axis, slot), x_end = quad_cut(axis, slot + 1);
  if (x_begin >= x_end) return;

  // ---- LDS of this group ----
  unsigned char* tiles = lds + grp * C::GROUP_TILES;
  const unsigned tiles_addr = (unsigned)(uintptr_t)(lds_ptr_t)lds + grp * C::GROUP_TILES;
  int32_t* lists = reinterpret_cast<int32_t*>(lds + C::OFF_LISTS) + grp * 3 * C::NB_CAP;   // ring of three lists
  int32_t* desc = reinterpret_cast<int32_t*>(lds + C::OFF_DESC) + grp * 3 * 8;             // and their descriptors

  const float qk_scale = prm.qk_scale;

  // per-lane LDS byte offsets of the operand reads (as fwd_kernel)
  int kaddr[2][KS];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int row = 32 * kb + ln;
      kaddr[kb][s] = row * ROWB + (((2 * s + g) ^ k_swz<D>(row)) * 16);
    }
  // the extra contraction slice that brings the reference exponent into the scores: ones x (-m_hi, -m_lo);
  // only the first of the four registers of either operand is not zero, and only it is kept
  const unsigned ones0 = g == 0 ? 0x3c003c00u : 0u;

  // This wavefront's share of a tile copy: instructions 2r and 2r + 1 of the eight (rows 16r .. 16r + 15)
  constexpr int RPI = 64 / CPR;      // tile rows per copy instruction (8)
  unsigned koff[2], voff[2];
#pragma unroll
  for (int jj = 0; jj < 2; ++jj) {
    const int row = (2 * r + jj) * RPI + lane / CPR, ch = lane % CPR;
    koff[jj] = 2u * (unsigned)(row * (CONTIG ? D : (int)prm.ks[2]) + ((ch ^ k_swz<D>(row)) * 8));
    voff[jj] = 2u * (unsigned)(row * prm.N + ((ch ^ k_swz<D>(row)) * 8));     // row = head-dimension index of V^T
  }
  const int64_t k_rs = CONTIG ? (int64_t)D : prm.ks[2];
  auto copy_k = [&](const unsigned short* kg, int cb, int buf) {
    const unsigned short* tile = kg + (int64_t)cb * 64 * k_rs;
    const unsigned dst = tiles_addr + buf * C::TILE_BYTES + 2 * r * 1024;
    tile_load_async_one(tile, koff[0], dst);
    tile_load_async_one(tile, koff[1], dst + 1024);
  };
  // (V comes from its transposed copy [head][64][N], see vt_kernel: a tile is 64 rows of 128 bytes, N elements apart)
  auto copy_v = [&](const unsigned short* vg, int cb, int buf) {
    const unsigned short* tile = vg + (int64_t)cb * 64;
    const unsigned dst = tiles_addr + (3 + buf) * C::TILE_BYTES + 2 * r * 1024;
    tile_load_async_one(tile, voff[0], dst);
    tile_load_async_one(tile, voff[1], dst + 1024);
  };

  // ---- state of the row block this wavefront is working on ----
  uintx4 qf[2][KS];
  floatx16 oacc[DB][2];
  float m_i[2], l_i[2];
  unsigned mfrag0[2];
  bool fresh = true;
  uintx4 pf[4][2];                  // numerators between the vector phase and the next matrix phase

  auto reset_acc = [&]() {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[db][qb][i] = 0.f;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) { m_i[qb] = 0.f; l_i[qb] = 0.f; mfrag0[qb] = 0u; }
    fresh = true;
  };
  // Q fragments of row block `row` of head (b, h); rows past the end of the sequence load row 0 (never used)
  auto load_q = [&](const unsigned short* qg, int row) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const unsigned short* qrow = qg + (int64_t)(row * 64 + qb * 32 + ln) * prm.qs[2];
#pragma unroll
      for (int s = 0; s < KS; ++s) qf[qb][s] = *reinterpret_cast<const uintx4*>(qrow + 16 * s + 8 * g);
    }
  };
  auto scale_q = [&]() {
    if constexpr (FOLD) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          const uintx4 raw = qf[qb][s];
          qf[qb][s] = uintx4{scale_half2(raw[0], qk_scale), scale_half2(raw[1], qk_scale),
                             scale_half2(raw[2], qk_scale), scale_half2(raw[3], qk_scale)};
        }
    }
  };

  // ---- the steps of a tile ----
  auto read_k = [&](const unsigned char* lds_k, uintx4 (&kfr)[2][KS]) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int s = 0; s < KS; ++s) kfr[kb][s] = *reinterpret_cast<const uintx4*>(lds_k + kaddr[kb][s]);
  };
  auto first_product = [&](const uintx4 (&kfr)[2][KS], floatx16& sa0, floatx16& sa1, floatx16& sb0, floatx16& sb1) {
    auto scores = [&](int qb, floatx16& s0, floatx16& s1) {
#pragma unroll
      for (int i = 0; i < 16; ++i) { s0[i] = 0.f; s1[i] = 0.f; }
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        s0 = mfma_qk<BF16>(kfr[0][s], qf[qb][s], s0);
        s1 = mfma_qk<BF16>(kfr[1][s], qf[qb][s], s1);
      }
      if constexpr (FOLD) {
        s0 = mfma_qk<BF16>(uintx4{ones0, 0u, 0u, 0u}, uintx4{mfrag0[qb], 0u, 0u, 0u}, s0);
        s1 = mfma_qk<BF16>(uintx4{ones0, 0u, 0u, 0u}, uintx4{mfrag0[qb], 0u, 0u, 0u}, s1);
      }
    };
    scores(0, sa0, sa1);
    scores(1, sb0, sb1);
  };
  // V^T fragment (ts, db): rows = head-dimension values 32 db + ln, keys 16 ts + 8 g .. + 8 in the order the
  // transposed copy stores them, which is the order the numerators leave the accumulators in: same
  // addresses as the K fragments
  auto read_v = [&](const unsigned char* lds_v, uintx4 (&vfr)[4][DB]) {
#pragma unroll
    for (int ts = 0; ts < 4; ++ts)
#pragma unroll
      for (int db = 0; db < DB; ++db) vfr[ts][db] = *reinterpret_cast<const uintx4*>(lds_v + kaddr[db][ts]);
  };
  auto second_product = [&](const uintx4 (&vfr)[4][DB]) {
#pragma unroll
    for (int ts = 0; ts < 4; ++ts)
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
          oacc[db][qb] = mfma_qk<PB>(vfr[ts][db], pf[ts][qb], oacc[db][qb]);
  };
  // Softmax numerators of one query block, in place: the scores are replaced by P = exp2(score - m)
  // (32 exponentials back to back, nothing waits for another), summed in fp32 before rounding as the
  // reference does (fa2_custom_mask/fa2_fwd.py:179; four independent chains), then rounded and packed as
  // the operand fragments pn[0..3][qb].  (The dot-product instruction that would add two rounded values
  // at once shares hardware with the matrix cores: beside the other group's MFMAs it costs twice the
  // two plain additions.)
  auto exp_pack = [&](int qb, floatx16& s0, floatx16& s1, uintx4 (&pn)[4][2]) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s0[i] = __builtin_amdgcn_exp2f(FOLD ? s0[i] : __builtin_fmaf(s0[i], qk_scale, -m_i[qb]));
      s1[i] = __builtin_amdgcn_exp2f(FOLD ? s1[i] : __builtin_fmaf(s1[i], qk_scale, -m_i[qb]));
    }
    float part[4] = {l_i[qb], 0.f, 0.f, 0.f};
#pragma unroll
    for (int ts = 0; ts < 4; ++ts)
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int i = 8 * (ts & 1) + 2 * jj;
        const float p0 = ts < 2 ? s0[i] : s1[i], p1 = ts < 2 ? s0[i + 1] : s1[i + 1];
        part[jj] += p0;
        part[jj] += p1;
        pn[ts][qb][jj] = pack2<PB>(p0, p1);
      }
    return (part[0] + part[1]) + (part[2] + part[3]);
  };
  // The scores of one query block again (the numerators have replaced them): the K tile is still in LDS.
  auto scores_again = [&](const unsigned char* lds_k, int qb, floatx16& s0, floatx16& s1) {
#pragma unroll
    for (int i = 0; i < 16; ++i) { s0[i] = 0.f; s1[i] = 0.f; }
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const uintx4 k0 = *reinterpret_cast<const uintx4*>(lds_k + kaddr[0][s]);
      const uintx4 k1 = *reinterpret_cast<const uintx4*>(lds_k + kaddr[1][s]);
      s0 = mfma_qk<BF16>(k0, qf[qb][s], s0);
      s1 = mfma_qk<BF16>(k1, qf[qb][s], s1);
    }
    if constexpr (FOLD) {
      s0 = mfma_qk<BF16>(uintx4{ones0, 0u, 0u, 0u}, uintx4{mfrag0[qb], 0u, 0u, 0u}, s0);
      s1 = mfma_qk<BF16>(uintx4{ones0, 0u, 0u, 0u}, uintx4{mfrag0[qb], 0u, 0u, 0u}, s1);
    }
  };
  auto numerators = [&](const unsigned char* lds_k, floatx16& sa0, floatx16& sa1, floatx16& sb0, floatx16& sb1, uintx4 (&pn)[4][2]) {
    auto one = [&](int qb, floatx16& s0, floatx16& s1) {
      float lnew = exp_pack(qb, s0, s1, pn);
      // Rare: the first tile of a row block, or some P left the safe fp16 range (the lane's sum grew by
      // 2^14 or more, or is not finite).  The reference exponent moves to the tile's row maximum and the
      // numerators are redone from the scores, which are computed once more.
      if (__builtin_expect(__any(fresh || !(lnew - l_i[qb] < 16384.0f)), 0)) {
        scores_again(lds_k, qb, s0, s1);
        uintx4 mf = {mfrag0[qb], 0u, 0u, 0u};
        recentre<DB, FOLD, false>(s0, s1, oacc, qb, qk_scale, m_i[qb], l_i[qb], mf, fresh, g);
        mfrag0[qb] = mf[0];
        lnew = exp_pack(qb, s0, s1, pn);
      }
      l_i[qb] = lnew;
    };
    one(0, sa0, sa1);
    one(1, sb0, sb1);
    fresh = false;
  };

  // ---- segments: the part of a quad's union list that falls into this group's range ----
  // descriptor of a ring entry (ints in LDS): 0 quad, 1 entries, 2 part index, 3 parts, 4 "is the
  // group's first segment".  List entry: column block | membership of the quad's rows << 16.
  int64_t x_cursor = x_begin;      // weight position up to which segments have been generated
  int built = 0;                   // segments generated so far
  auto build_next = [&]() {        // generates segment number `built` into ring entry built % 3 (n = 0: no more)
    int32_t* d = desc + (built % 3) * 8;
    int32_t* dst = lists + (built % 3) * C::NB_CAP;
    if (x_cursor >= x_end) { if (lane == 0) d[1] = 0; ++built; return; }
    const QuadPos qp = quad_locate(axis, x_cursor);
    const int64_t seg_end = x_end < qp.c0 + qp.w ? x_end : qp.c0 + qp.w;
    // (a quad's weight is the size of its union list: weight offsets are list positions)
    const int o0 = (int)(x_cursor - qp.c0), o1 = (int)(seg_end - qp.c0);
    const QuadParts parts = quad_parts(axis, qp.c0, qp.w);
    const int32_t* src = prm.quad_list + (int64_t)(shared_mask ? qp.gq % nq : qp.gq) * nb + o0;
    for (int i = lane; i < o1 - o0; i += 64) dst[i] = src[i];
    if (lane == 0) {
      d[0] = qp.gq; d[1] = o1 - o0; d[2] = slot - parts.first; d[3] = parts.count; d[4] = built == 0;
      d[5] = (int)(unsigned)(qp.c0 & 0xffffffffll); d[6] = (int)(qp.c0 >> 32);
    }
    x_cursor = seg_end;
    ++built;
  };
  auto desc_get = [&](int seg, int field) { return __builtin_amdgcn_readfirstlane(desc[(seg % 3) * 8 + field]); };
  auto list_get = [&](int seg, int pos) { return __builtin_amdgcn_readfirstlane(lists[(seg % 3) * C::NB_CAP + pos]); };

  // ---- finishing a row block ----
  const int64_t part_floats = partial_floats(D);
  // part (slot s, first / later segment, row of the quad)
  auto part_ptr = [&](int s, int which, int rr) { return prm.ws + (((int64_t)s * 2 + which) * 4 + rr) * part_floats; };
  auto write_rowblock = [&](int bh, int row, const float (&L)[2], const float (&M)[2]) {
    const int b = bh / prm.H, h = bh - b * prm.H;
    void* obase = out_base(prm, b, h);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const float inv = L[qb] > 0.f ? 1.0f / L[qb] : 0.f;
      const int64_t qrow = (int64_t)(row * 64 + qb * 32 + ln);
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4)
          store_out4<BF16>(obase, qrow * prm.os[2] + 32 * db + 8 * i4 + 4 * g, prm.out_f32,
                           oacc[db][qb][4 * i4] * inv, oacc[db][qb][4 * i4 + 1] * inv,
                           oacc[db][qb][4 * i4 + 2] * inv, oacc[db][qb][4 * i4 + 3] * inv);
      if (prm.lse != nullptr && g == 0)
        prm.lse[(int64_t)bh * prm.N + qrow] =
            L[qb] > 0.f ? (M[qb] + __builtin_amdgcn_logf(L[qb])) * 0.6931471805599453f : -INFINITY;
    }
  };
  // had_tiles: this wavefront processed at least one tile of the segment
  auto finish_rowblock = [&](int seg, bool had_tiles) {
    const int gq = desc_get(seg, 0), part = desc_get(seg, 2), nparts = desc_get(seg, 3), which = desc_get(seg, 4) ? 0 : 1;
    const int bh = gq / nq, qi = gq - bh * nq, row = 4 * qi + r;
    if (row >= nb) return;
    const int32_t* rpm = prm.row_ptr + (int64_t)(shared_mask ? 0 : bh) * nb;
    if (__builtin_amdgcn_readfirstlane(rpm[row + 1]) == __builtin_amdgcn_readfirstlane(rpm[row])) return;   // written by the sweep above
    float L[2], M[2];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) { L[qb] = l_i[qb] + __shfl_xor(l_i[qb], 32); M[qb] = m_i[qb]; }
    if (__builtin_expect(nparts == 1, 1)) { write_rowblock(bh, row, L, M); return; }
    // publish this part: [16 quads of registers][lane][4] floats, then m[64], l[64]
    float* mine = part_ptr(slot, which, r);
    if (had_tiles) {
#pragma unroll
      for (int i4 = 0; i4 < 16; ++i4) {
        const int idx = 4 * i4;
        const floatx4 v = {oacc[idx / 32][(idx / 16) & 1][idx & 15], oacc[idx / 32][(idx / 16) & 1][(idx & 15) + 1],
                           oacc[idx / 32][(idx / 16) & 1][(idx & 15) + 2], oacc[idx / 32][(idx / 16) & 1][(idx & 15) + 3]};
        coherent_store4(mine + (i4 * 64 + lane) * 4, v);
      }
    }
    if (g == 0) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        const bool mass = had_tiles && L[qb] > 0.f;
        coherent_store(mine + 64 * D + qb * 32 + ln, mass ? M[qb] : -INFINITY);
        coherent_store(mine + 64 * D + 64 + qb * 32 + ln, mass ? L[qb] : 0.f);
      }
    }
    wait_vm<0>();        // the stores have been acknowledged
    // count this part in: the counter holds (launch mark << 16 | parts arrived); stale contents carry another mark
    unsigned long long* ctr = prm.qcounters + (int64_t)bh * nb + row;
    int arrived = 0;
    if (lane == 0) {
      unsigned long long old = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      for (;;) {
        const unsigned long long want = (old >> 16) == prm.epoch ? old + 1 : ((prm.epoch << 16) | 1ull);
        if (__hip_atomic_compare_exchange_strong(ctr, &old, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
          arrived = (int)(want & 0xffffull);
          break;
        }
      }
    }
    arrived = __builtin_amdgcn_readfirstlane(arrived);
    asm volatile("" ::: "memory");
    if (__builtin_expect(arrived != nparts, 1)) return;
    // last to arrive: all parts are in memory.  Sum them in part order.
    const int s0 = slot - part;      // range that holds part 0
    const int64_t c0 = (int64_t)(unsigned)desc_get(seg, 5) | ((int64_t)desc_get(seg, 6) << 32);
    const bool part0_first = quad_cut(axis, s0) == c0;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[db][qb][i] = 0.f;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) { M[qb] = -INFINITY; L[qb] = 0.f; }
    for (int p = 0; p < nparts; ++p) {
      // part 0 is a later segment of its range unless that range starts with this quad; the others start inside the quad
      const int wh = p == part ? which : (p == 0 ? (part0_first ? 0 : 1) : 0);
      const float* src = part_ptr(s0 + p, wh, r);
      float mp[2], lp[2];
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        mp[qb] = coherent_load(src + 64 * D + qb * 32 + ln);
        lp[qb] = coherent_load(src + 64 * D + 64 + qb * 32 + ln);
      }
      if (!__any(lp[0] > 0.f || lp[1] > 0.f)) continue;     // a part without tiles
      floatx4 dat[16];
#pragma unroll
      for (int i4 = 0; i4 < 16; ++i4) dat[i4] = coherent_load4(src + (i4 * 64 + lane) * 4);
      asm volatile("s_waitcnt vmcnt(0)"
                   : "+v"(dat[0]), "+v"(dat[1]), "+v"(dat[2]), "+v"(dat[3]), "+v"(dat[4]), "+v"(dat[5]), "+v"(dat[6]), "+v"(dat[7]),
                     "+v"(dat[8]), "+v"(dat[9]), "+v"(dat[10]), "+v"(dat[11]), "+v"(dat[12]), "+v"(dat[13]), "+v"(dat[14]), "+v"(dat[15])
                   :: "memory");
      float so[2], sp[2];
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        const float mn = fmaxf(M[qb], mp[qb]);
        so[qb] = M[qb] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(M[qb] - mn);
        sp[qb] = mp[qb] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mp[qb] - mn);
        L[qb] = L[qb] * so[qb] + lp[qb] * sp[qb];
        M[qb] = mn;
      }
#pragma unroll
      for (int i4 = 0; i4 < 16; ++i4) {
        const int idx = 4 * i4, db = idx / 32, qb = (idx / 16) & 1;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          oacc[db][qb][(idx & 15) + e] = oacc[db][qb][(idx & 15) + e] * so[qb] + dat[i4][e] * sp[qb];
      }
    }
    write_rowblock(bh, row, L, M);
    // the counter goes back to zero, so that a replay of this launch (same mark) starts clean
    if (lane == 0) __hip_atomic_store(ctr, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };

  // =========================== prologue ===========================
  build_next();     // segment 0
  build_next();     // segment 1
  const unsigned short *qg = nullptr, *kg = nullptr, *vg = nullptr;
  auto enter_segment = [&](int s) {           // head pointers of the segment's quad
    const int gq = desc_get(s, 0);
    const int bh = gq / nq, b = bh / prm.H, h = bh - b * prm.H;
    qg = (const unsigned short*)prm.q + b * prm.qs[0] + h * prm.qs[1];
    kg = (const unsigned short*)prm.k + b * prm.ks[0] + h * prm.ks[1];
    vg = prm.vt + (int64_t)bh * 64 * prm.N;
    return 4 * (gq - bh * nq) + r;            // this wavefront's row block
  };
  auto head_k = [&](int s) {
    const int gq = desc_get(s, 0); const int bh = gq / nq, b = bh / prm.H, h = bh - b * prm.H;
    return (const unsigned short*)prm.k + b * prm.ks[0] + h * prm.ks[1];
  };
  int my_row = enter_segment(0);
  load_q(qg, my_row < nb ? my_row : 0);
  reset_acc();
  copy_k(kg, list_get(0, 0) & 0xffff, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): Q and this wavefront's share of the first K tile
  scale_q();
  // A phase ends at a workgroup barrier.  Nothing may be moved across it: not the LDS accesses (fences)
  // and not the matrix and vector instructions either (the phases exist to keep them apart).
  auto sync = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- state of the walk ----
  int t = 0;                    // tiles of this group so far (V buffer parity)
  int kt = 0;                   // t % 3 (K buffer: three of them, because the numerators may read the K tile again while
                                // the copy for the round after next is already on its way)
  int seg = 0;                  // current segment, and what is known about it:
  int n = 0;                    //   its tiles
  bool more = false;            //   another segment follows
  const unsigned short* kg_next = nullptr;   // K of the head of the next segment
  int first_next = -1;          //   and the column block of its first tile (-1: none)
  const int32_t* list = nullptr;
  int entry = 0;                // list entry of the tile of the coming round
  int col_next = -1;            // column block of the tile after that one (-1: none)
  auto setup_segment = [&](int sg) {
    seg = sg;
    n = desc_get(sg, 1);
    more = desc_get(sg + 1, 1) > 0;
    kg_next = more ? head_k(sg + 1) : kg;
    first_next = more ? list_get(sg + 1, 0) & 0xffff : -1;
    list = lists + (sg % 3) * C::NB_CAP;
    entry = list_get(sg, 0);
    col_next = n > 1 ? list_get(sg, 1) & 0xffff : first_next;
  };
  // Copies for the rounds to come, started at the end of a vector phase: the K tile of the round after
  // next (whose first product is two barriers away) and the V tile of the next round (whose second product
  // is).  Both buffers were last read in the matrix phase that has just ended.
  auto copies_ahead = [&](bool k_in_segment) {
    if (col_next >= 0) copy_k(k_in_segment ? kg : kg_next, col_next, kt == 2 ? 0 : kt + 1);
    copy_v(vg, entry & 0xffff, t & 1);
  };
  setup_segment(0);
  copies_ahead(n > 1);
  sync();                                 // the first K tile is complete
  if (grp == 1) sync();                   // the second group runs one phase behind the first
  QUAD_WALL(1);

  // =========================== segments ===========================
  for (;;) {
    bool p_live = false, had_tiles = false;
    // One tile.  Matrix phase: operand fragments from LDS, the second product of the previous tile, the first
    // product of this one; barrier.  Vector phase: numerators; the copies started a round ago are waited for
    // and the copies for later rounds started; barrier.
    auto round = [&](int pos, auto last_tag) {
      constexpr bool LAST = decltype(last_tag)::value;
      const bool mine = (entry >> (16 + r)) & 1;
      const unsigned char* lds_k = tiles + kt * C::TILE_BYTES;
      uintx4 vfr[4][DB], kfr[2][KS];
      // (read whether needed or not: a wavefront that sits the tile out ignores what it gets)
      read_v(tiles + (3 + ((t - 1) & 1)) * C::TILE_BYTES, vfr);
      read_k(lds_k, kfr);
      // all sixteen reads are on their way before the first MFMA waits for one (left to itself the compiler
      // reads the V fragments one at a time into one register group, each read a full LDS round trip in
      // front of two MFMAs)
      __builtin_amdgcn_sched_barrier(0);
      if (p_live) { second_product(vfr); p_live = false; }
      // list entries of the next round (picked up in the vector phase)
      int raw_entry = 0, raw_next = 0;
      if (!LAST) {
        raw_entry = list[pos + 1];
        raw_next = pos + 2 < n ? list[pos + 2] : 0;
      }
      if (mine) {
        // the scores live from the matrix phase to the vector phase of this round only
        floatx16 sa0, sa1, sb0, sb1;
        first_product(kfr, sa0, sa1, sb0, sb1);
        had_tiles = true;
        sync();
        numerators(lds_k, sa0, sa1, sb0, sb1, pf);
        p_live = true;
      } else {
        sync();
      }
      ++t;
      kt = kt == 2 ? 0 : kt + 1;
      if (LAST) {
        if (more) {
          // Q of the next segment's row block (the fragments of this one are not needed any more)
          my_row = enter_segment(seg + 1);
          load_q(qg, my_row < nb ? my_row : 0);
        }
      } else {
        entry = __builtin_amdgcn_readfirstlane(raw_entry);
        col_next = pos + 2 < n ? (__builtin_amdgcn_readfirstlane(raw_next) & 0xffff) : first_next;
      }
      wait_vm<0>();            // this wavefront's shares of the copies started a round ago (LAST: and Q)
      if (!LAST) copies_ahead(pos + 2 < n);
      sync();
    };
    for (int pos = 0; pos + 1 < n; ++pos) round(pos, std::false_type{});
    round(n - 1, std::true_type{});
    // ---- the owed second product, in a matrix phase of its own; then the row block is complete ----
    if (p_live) {
      uintx4 vfr[4][DB];
      read_v(tiles + (3 + ((t - 1) & 1)) * C::TILE_BYTES, vfr);
      second_product(vfr);
    }
    if (!more) QUAD_WALL(2);
    finish_rowblock(seg, had_tiles);
    if (!more) QUAD_WALL(3);
    if (!more) return;
    __builtin_amdgcn_s_waitcnt(0x0F70);   // (Q, and whatever finishing the row block left in flight)
    sync();
    build_next();                         // segment seg + 2 (ring of three: seg + 1 is in use next)
    setup_segment(seg + 1);
    reset_acc();
    scale_q();
    // (everything in flight is waited for here, where the compiler sees it: inside the rounds no wait of its
    // making may sit between the asynchronous tile copies)
    __builtin_amdgcn_s_waitcnt(0x0F70);
    copies_ahead(n > 1);
    sync();
  }
}

// V transposed for the second product: vt[head][d][p(n)] = v[head][n][d], 16-bit values, where p swaps
// bits 2 and 3 of the key index n.  With that order the eight keys a lane contributes to a
// contraction slice lie next to each other, and a V^T operand fragment is one 16-byte LDS read, like a
// K fragment.  TO_F16: bf16 input, fp16 output (the second product then runs in fp16 with P kept to
// 11 bits).  One workgroup per 64 keys of a head.
template <bool TO_F16>
__global__ __launch_bounds__(256) void vt_kernel(const unsigned short* __restrict__ v, unsigned short* __restrict__ vt,
                                                 int H, int N, int64_t sb, int64_t sh, int64_t sn) {
  __shared__ unsigned short tile[64][66];
  const int bh = blockIdx.y, b = bh / H, h = bh - b * H, n0 = blockIdx.x * 64;
  const unsigned short* src = v + b * sb + h * sh + (int64_t)n0 * sn;
  // 64 keys x 64 values in, 8 values per thread
  for (int i = threadIdx.x; i < 64 * 8; i += 256) {
    const int n = i >> 3, c = i & 7;
    const uintx4 x = *reinterpret_cast<const uintx4*>(src + (int64_t)n * sn + 8 * c);
    const int pn = (n & ~12) | ((n & 4) << 1) | ((n & 8) >> 1);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      unsigned lo = x[e] & 0xffffu, hi = x[e] >> 16;
      if (TO_F16) {
        const half2v hh = {(_Float16)__builtin_bit_cast(float, lo << 16), (_Float16)__builtin_bit_cast(float, hi << 16)};
        const unsigned u = __builtin_bit_cast(unsigned, hh);
        lo = u & 0xffffu; hi = u >> 16;
      }
      tile[8 * c + 2 * e][pn] = (unsigned short)lo;
      tile[8 * c + 2 * e + 1][pn] = (unsigned short)hi;
    }
  }
  __syncthreads();
  unsigned short* dst = vt + (int64_t)bh * 64 * N + n0;
  for (int i = threadIdx.x; i < 64 * 32; i += 256) {
    const int d = i >> 5, c = i & 31;       // 2 keys per thread: 128 contiguous bytes per row
    const unsigned w = (unsigned)tile[d][2 * c] | ((unsigned)tile[d][2 * c + 1] << 16);
    *reinterpret_cast<unsigned*>(dst + (int64_t)d * N + 2 * c) = w;
  }
}

// bytes of the transposed V copy
size_t quad_vt_bytes(int B, int H, int N) { return (size_t)B * H * N * 64 * 2; }

// workspace: parts [slots][2][4][partial_floats], counters [B*H*nb], transposed V
size_t quad_parts_bytes(int slots) { return (size_t)slots * 2 * 4 * partial_floats(64) * sizeof(float); }
size_t quad_counters_bytes(int B, int H, int nb) { return (((size_t)B * H * nb * sizeof(unsigned long long)) + 255) & ~(size_t)255; }
size_t quad_workspace_bytes(int slots, int B, int H, int nb) {
  return quad_parts_bytes(slots) + quad_counters_bytes(B, H, nb) + quad_vt_bytes(B, H, nb * 64);
}

bool quad_supported(const AttnShape& s) {
  const int nb = s.N / 64, nq = (nb + 3) / 4;
  if (s.D != 64 || nb > QuadCfg::NB_CAP) return false;
  const bool shared = s.Bm == 1 && s.Hm == 1, full = s.Bm == s.B && s.Hm == s.H;
  if (!shared && !full) return false;
  const int64_t period = shared ? nq : (int64_t)s.B * s.H * nq;
  return period <= QuadCfg::CUM_CAP;
}

template <int DT, bool CONTIG>
static void launch_quad_t(const FwdParams& prm, int wgs, hipStream_t st) {
  static std::atomic<unsigned long long> configured{0};
  once_per_device(configured, [] {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&fwd_quad_kernel<DT, CONTIG>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, QuadCfg::LDS_BYTES);
  });
  hipLaunchKernelGGL((fwd_quad_kernel<DT, CONTIG>), dim3(wgs), dim3(512), QuadCfg::LDS_BYTES, st, prm);
}

void launch_fwd_quad(const FwdParams& prm, int dt, hipStream_t st) {
  {
    const dim3 grid(prm.nb, prm.B * prm.H);
    const unsigned short* v = (const unsigned short*)prm.v;
    unsigned short* vt = const_cast<unsigned short*>(prm.vt);
    if (dt == 1) hipLaunchKernelGGL(vt_kernel<true>, grid, dim3(256), 0, st, v, vt, prm.H, prm.N, prm.vs[0], prm.vs[1], prm.vs[2]);
    else hipLaunchKernelGGL(vt_kernel<false>, grid, dim3(256), 0, st, v, vt, prm.H, prm.N, prm.vs[0], prm.vs[1], prm.vs[2]);
  }
  const bool contig = prm.ks[2] == 64;
  const int wgs = prm.qslots / 2;
  if (contig) {
    if (dt == 0) launch_quad_t<0, true>(prm, wgs, st); else if (dt == 1) launch_quad_t<1, true>(prm, wgs, st); else launch_quad_t<2, true>(prm, wgs, st);
  } else {
    if (dt == 0) launch_quad_t<0, false>(prm, wgs, st); else if (dt == 1) launch_quad_t<1, false>(prm, wgs, st); else launch_quad_t<2, false>(prm, wgs, st);
  }
}

}  // namespace bsattn
