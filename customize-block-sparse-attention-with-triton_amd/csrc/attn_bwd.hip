// Block-sparse FlashAttention-2 backward for gfx950.
//
// Gradient algebra of the reference (fa2_custom_mask/fa2_bwd.py:17,57-74,117-130,232,284),
// evaluated over exactly the kept tiles:
//   delta = rowsum(O * dO);  P = exp(S*sm_scale - lse);  dV = P^T dO;  dP = dO V^T;
//   dS = P * (dP - delta);   dK = sm_scale * dS^T Q;     dQ = sm_scale * dS K.
// Two kernels, no atomics, results independent of scheduling:
//   dq_kernel     one workgroup (2 wavefronts x 32 queries) per row block, walking the row
//                 lists: per kept tile  S^T = K Q^T,  dP^T = V dO^T,  dQ^T += K^T dS^T;
//                 it also computes delta of its queries on the way in (dO is in its registers
//                 anyway) and leaves it in the workspace for the next kernel;
//   dkdv_kernel   one workgroup (2 wavefronts x 32 keys) per column block, walking the column
//                 lists: per kept tile  S = Q K^T,  dP = dO V^T,  dV^T += dO^T P,  dK^T += Q^T dS.
// Operand roles are chosen so that the fragment a wavefront owns for the whole walk (Q, dO or
// K, V) sits along the lanes: the per-row scalars (lse, delta) are then per-lane values in
// dq_kernel, P and dS leave the first products already in the operand layout of the second
// ones, and the tiles that change per step are staged in LDS by asynchronous copies into a
// double buffer (one barrier per tile).
#include "common.h"
#include "kernel_util.h"
#include <type_traits>

namespace bsattn {

struct BwdParams {
  const void* q; const void* k; const void* v; const void* o; const void* d_o;
  const float* lse; float* delta;
  void* dq; void* dk; void* dv;
  const int32_t* row_ptr; const int32_t* col_idx; const int32_t* col_ptr; const int32_t* row_idx;
  // elementwise masks: 64 words per entry of the row lists (bit = key) / of the column lists (bit = query)
  const unsigned long long* bits_rows; const unsigned long long* bits_cols;
  int B, H, N, nb, Bm, Hm;
  int out_f32;
  int split;                  // workgroups per row / column list (1: results written directly)
  float* part_dq; float* part_dk; float* part_dv;   // split > 1: fp32 partial results [split][B*H][N][D]
  float sm_scale, qk_scale;   // qk_scale = sm_scale * log2(e)
  int64_t qs[3], ks[3], vs[3], os[3], dos[3];
  int64_t dqs[3], dks[3], dvs[3];   // batch, head, row strides of the results (elements)
};

constexpr float kLog2e = 1.4426950408889634f;

// sum of the products of the eight 16-bit elements of a and b
template <bool BF16>
__device__ __forceinline__ float dot8(const uintx4& a, const uintx4& b, float acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float a0, a1, b0, b1;
    const unsigned int au = a[i], bu = b[i];   // by value: bit_cast of a vector element lvalue miscompiles
    if constexpr (BF16) {
      a0 = __builtin_bit_cast(float, au << 16); a1 = __builtin_bit_cast(float, au & 0xffff0000u);
      b0 = __builtin_bit_cast(float, bu << 16); b1 = __builtin_bit_cast(float, bu & 0xffff0000u);
    } else {
      const half2v ah = __builtin_bit_cast(half2v, au), bhh = __builtin_bit_cast(half2v, bu);
      a0 = (float)ah[0]; a1 = (float)ah[1]; b0 = (float)bhh[0]; b1 = (float)bhh[1];
    }
    acc += a0 * b0 + a1 * b1;
  }
  return acc;
}

// ---------------------------------------------------------------------------------------
// helpers of the two walking kernels
// ---------------------------------------------------------------------------------------
// ROWS: rows of a tile staged per step (64, or 32 when a tile is walked in two halves)
template <int D, bool EW, int ROWS = 64> struct BwdCfg {
  static constexpr int TILE_BYTES = ROWS * 2 * D;
  static constexpr int STAT_BYTES = 2 * 64 * 4;                    // lse2[64] + delta[64] of a row block
  static constexpr int BITS_BYTES = EW ? 64 * 8 : 0;               // mask words of the tile (elementwise masks)
  static constexpr int STAGE_BYTES = 2 * TILE_BYTES + STAT_BYTES + BITS_BYTES;  // two tiles, row statistics, mask words
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;                // double buffer
};

// This wavefront's half of the asynchronous copy of a ROWS x D tile (rows `stride` elements apart)
// into LDS with the u_swz chunk swizzle: wavefront wv issues half of the ROWS*D/512 instructions.
template <int D, int ROWS = 64>
__device__ __forceinline__ void half_tile_load_async(const unsigned short* tile, int64_t stride, int wv, int lane,
                                                     unsigned lds_addr) {
  constexpr int CPR = D / 8, PER_WAVE = ROWS * CPR / 128;
#pragma unroll
  for (int jj = 0; jj < PER_WAVE; ++jj) {
    const int j = wv * PER_WAVE + jj;
    const int c = j * 64 + lane, row = c / CPR, ch = c % CPR;
    const unsigned off = 2u * (unsigned)(row * (int)stride + ((ch ^ u_swz<D>(row)) * 8));
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_addr + j * 1024), "v"(off), "s"(tile) : "memory", "m0");
  }
}

// asynchronous copy of 64 consecutive floats (one per lane)
__device__ __forceinline__ void stat_load_async(const float* src, int lane, unsigned lds_addr) {
  const unsigned off = 4u * (unsigned)lane;
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2" :: "s"(lds_addr), "v"(off), "s"(src) : "memory", "m0");
}

// operand fragment (32 rows x 16 columns slice s) of a swizzled LDS tile: row r0 + ln, chunk 2s + g
template <int D>
__device__ __forceinline__ uintx4 frag_rows(const unsigned char* tile, int r0, int s, int ln, int g) {
  const int row = r0 + ln;
  return *reinterpret_cast<const uintx4*>(tile + row * 2 * D + (((2 * s + g) ^ u_swz<D>(row)) * 16));
}

// transposed operand fragment: columns 32db + ln of the tile along the lanes, contraction slots j
// of slice ts <-> tile rows 16ts + 8(j/4) + 4g + (j%4) (the order in which a 32x32 MFMA result
// holds its rows), by two LDS transpose reads
template <int D, bool BF16>
__device__ __forceinline__ uintx4 frag_cols(const unsigned char* tile, int db, int ts, int lane) {
  const int blk = lane >> 4, s16 = lane & 15;
  uintx4 a;
#pragma unroll
  for (int jh = 0; jh < 2; ++jh) {
    const int row = 16 * ts + 8 * jh + 4 * (blk >> 1) + (s16 >> 2);
    const int col = 32 * db + 16 * (blk & 1) + 4 * (s16 & 3);
    const int addr = row * 2 * D + (((col >> 3) ^ u_swz<D>(row)) * 16) + (col & 7) * 2;
    const short4v rr = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(tile + addr));
    const uintx2 r2 = __builtin_bit_cast(uintx2, rr);
    a[2 * jh] = r2[0]; a[2 * jh + 1] = r2[1];
  }
  if constexpr (BF16) a = bf16x8_to_f16x8(a);
  return a;
}

// scores of unset mask elements become -inf; mw: the 64 mask bits of this lane's row, already
// shifted right by 4 g, so that bit 8(i/4) + i%4 (+ 32 for the second block) belongs to register i
__device__ __forceinline__ void mask_scores(floatx16& s0, floatx16& s1, unsigned long long mw) {
  const unsigned lo = (unsigned)mw, hi = (unsigned)(mw >> 32);
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const unsigned bit = 1u << (8 * (i / 4) + (i % 4));
    s0[i] = (lo & bit) ? s0[i] : -INFINITY;
    s1[i] = (hi & bit) ? s1[i] : -INFINITY;
  }
}

// the same for one block of 32 keys (bits 0..31 of the shifted word)
__device__ __forceinline__ void mask_scores(floatx16& s0, unsigned lo) {
#pragma unroll
  for (int i = 0; i < 16; ++i) s0[i] = (lo & (1u << (8 * (i / 4) + (i % 4)))) ? s0[i] : -INFINITY;
}

__device__ __forceinline__ floatx16 zero16() {
  floatx16 z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.f;
  return z;
}


// Values that live in registers through a walking loop (fragments of the stationary operand, row statistics) are
// passed through here once they have been asked for: the compiler waits for their loads at this point.  Left to
// itself it moves the loads next to the loop and plants its waits at their first uses inside it, where, being
// counted waits, they also wait for the tile copies of the next step that have just been issued, in every step.
__device__ __forceinline__ void settle(uintx4& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void settle(float& x) { asm volatile("" : "+v"(x)); }

// Workgroup -> (head, block) for the walking kernels.  Workgroups go to the 8 XCDs round-robin by
// linear id, and each XCD has its own L2: heads are taken in groups of 8, head i of a group on
// XCD i, so that the tiles a head's workgroups walk over (K and V, or Q and dO, of that head) are
// shared in one L2 instead of being fetched into all of them.
__device__ __forceinline__ void head_and_block(int L, int BH, int nb, int& bh, int& blk) {
  const int grp = L / (8 * nb), l = L - grp * 8 * nb;
  const int hg = BH - 8 * grp < 8 ? BH - 8 * grp : 8;     // heads in this group
  bh = 8 * grp + l % hg;
  blk = l / hg;          // >= nb for the padding of an incomplete last group
}

// ---------------------------------------------------------------------------------------
// dQ: workgroup = row block m, wavefront wv owns queries 64m + 32wv + ln
// ---------------------------------------------------------------------------------------
// PB (bf16 inputs only): dS is rounded to bf16 and the second product runs in bf16 on the tile as it
// is; otherwise dS is rounded to fp16 and bf16 tiles are converted fragment by fragment.
// KB: 32-key blocks of a tile handled per step.  2: a whole tile per step.  1 (used at D = 128): a
// tile is walked in two steps of 32 keys; the staged halves are 8 KB, four workgroups fit a compute
// unit and the wavefront stays within 256 registers: two wavefronts per SIMD.
template <int D, bool BF16, bool EW, bool PB, int KB>
__global__ __launch_bounds__(128, D == 256 ? 1 : 2) void dq_kernel(const BwdParams prm) {
  using C = BwdCfg<D, EW, 32 * KB>;
  constexpr int KS = D / 16, DB = D / 32, STEPS = 2 / KB;
  constexpr int PORTIONS = D == 256 ? 2 : 1, KSP = KS / PORTIONS;   // D = 256: the fragments of the first products in two portions
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ln = lane & 31, g = lane >> 5;
  const int nb = prm.nb;
  int bh, blk;
  const int per_chunk = gridDim.x / prm.split;               // chunk = slowest index: head i of a group stays on XCD i
  const int chunk = blockIdx.x / per_chunk;
  head_and_block(blockIdx.x - chunk * per_chunk, prm.B * prm.H, nb, bh, blk);
  if (blk >= nb) return;
  const int m = nb - 1 - blk;                 // long rows of block-causal masks first
  const int b = bh / prm.H, h = bh % prm.H;
  const int mh = (prm.Bm > 1 ? b : 0) * prm.Hm + (prm.Hm > 1 ? h : 0);
  const cint_ptr_t rp = (cint_ptr_t)(uintptr_t)(prm.row_ptr + (int64_t)mh * nb);
  const cint_ptr_t cols = (cint_ptr_t)(uintptr_t)prm.col_idx;
  // The rows this workgroup owns for its whole walk (Q, dO, O, lse of its queries) depend on the block index only:
  // they are asked for first, and travel while the list is looked up and the first tiles are requested.
  const int64_t qrow = (int64_t)m * 64 + 32 * wv + ln;
  const unsigned short* qp = (const unsigned short*)prm.q + b * prm.qs[0] + h * prm.qs[1] + qrow * prm.qs[2];
  const unsigned short* gp = (const unsigned short*)prm.d_o + b * prm.dos[0] + h * prm.dos[1] + qrow * prm.dos[2];
  const unsigned short* op = (const unsigned short*)prm.o + b * prm.os[0] + h * prm.os[1] + qrow * prm.os[2];
  uintx4 qfr[KS], dofr[KS], ofr[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    qfr[s] = *reinterpret_cast<const uintx4*>(qp + 16 * s + 8 * g);
    dofr[s] = *reinterpret_cast<const uintx4*>(gp + 16 * s + 8 * g);
  }
#pragma unroll
  for (int s = 0; s < KS; ++s) ofr[s] = *reinterpret_cast<const uintx4*>(op + 16 * s + 8 * g);
  const float lse_q = prm.lse[(int64_t)bh * prm.N + qrow];
  int u0, u1;                                                  // steps: tile u / STEPS, part u % STEPS
  {
    const int t0 = rp[m], len = rp[m + 1] - t0;                // this workgroup's share of the row's list
    u0 = (t0 + (int)((int64_t)len * chunk / prm.split)) * STEPS;
    u1 = (t0 + (int)((int64_t)len * (chunk + 1) / prm.split)) * STEPS;
  }
  const unsigned lds_addr = (unsigned)(uintptr_t)(lds_ptr_t)lds;

  const unsigned short* kg = (const unsigned short*)prm.k + b * prm.ks[0] + h * prm.ks[1];
  const unsigned short* vg = (const unsigned short*)prm.v + b * prm.vs[0] + h * prm.vs[1];
  auto issue = [&](int u, int stage) {
    const int t = u / STEPS;
    const int64_t key0 = (int64_t)cols[t] * 64 + (u % STEPS) * 32 * KB;
    half_tile_load_async<D, 32 * KB>(kg + key0 * prm.ks[2], prm.ks[2], wv, lane, lds_addr + stage * C::STAGE_BYTES);
    half_tile_load_async<D, 32 * KB>(vg + key0 * prm.vs[2], prm.vs[2], wv, lane,
                                     lds_addr + stage * C::STAGE_BYTES + C::TILE_BYTES);
    if constexpr (EW)   // the tile's 64 mask words, 256 bytes per wavefront
      stat_load_async(reinterpret_cast<const float*>(prm.bits_rows + (int64_t)t * 64) + wv * 64, lane,
                      lds_addr + stage * C::STAGE_BYTES + 2 * C::TILE_BYTES + C::STAT_BYTES + wv * 256);
  };
  if (u0 < u1) issue(u0, 0);

  // a query without any unmasked key has lse = -inf: every P of its row must come out as 0
  float lse2 = EW && lse_q == -INFINITY ? INFINITY : lse_q * kLog2e;
  // delta = rowsum(O * dO) (fa2_bwd.py:17): the lane holds one half of its query's row of dO, its neighbour 32
  // lanes on the other half.  Also kept for the dK/dV kernel, which needs it by key tile.
  float dlt;
  {
    float acc = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s) acc = dot8<BF16>(ofr[s], dofr[s], acc);
    dlt = acc + __shfl_xor(acc, 32);
    if (chunk == 0 && g == 0) prm.delta[(int64_t)bh * prm.N + qrow] = dlt;
  }
#pragma unroll
  for (int s = 0; s < KS; ++s) { settle(qfr[s]); settle(dofr[s]); }
  settle(lse2); settle(dlt);       // everything above has arrived: no vector-memory waits in the loop
  const float qk_scale = prm.qk_scale;

  floatx16 dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) dqacc[db] = zero16();

  for (int u = u0; u < u1; ++u) {
    const int stage = (u - u0) & 1;
    wait_vm<0>();
    __syncthreads();   // step u complete in `stage`; everyone is done with the other stage
    if (u + 1 < u1) issue(u + 1, stage ^ 1);
    const unsigned char* kt = lds + stage * C::STAGE_BYTES;
    const unsigned char* vt = kt + C::TILE_BYTES;

    // All operand fragments of a block of MFMAs are read from LDS before the block starts: a read
    // issued next to the MFMA that consumes it costs a full LDS latency per MFMA.
    floatx16 sacc[KB], dpacc[KB];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) { sacc[kb] = zero16(); dpacc[kb] = zero16(); }
#pragma unroll
    for (int pt = 0; pt < PORTIONS; ++pt) {
      uintx4 fk[KB][KSP], fv[KB][KSP];
#pragma unroll
      for (int s = 0; s < KSP; ++s)
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          fk[kb][s] = frag_rows<D>(kt, 32 * kb, pt * KSP + s, ln, g);
          fv[kb][s] = frag_rows<D>(vt, 32 * kb, pt * KSP + s, ln, g);
        }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < KSP; ++s)
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          sacc[kb] = mfma_qk<BF16>(fk[kb][s], qfr[pt * KSP + s], sacc[kb]);      // S^T = K Q^T
          dpacc[kb] = mfma_qk<BF16>(fv[kb][s], dofr[pt * KSP + s], dpacc[kb]);   // dP^T = V dO^T
        }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (EW) {
      unsigned long long mw = *reinterpret_cast<const unsigned long long*>(
          vt + C::TILE_BYTES + C::STAT_BYTES + (32 * wv + ln) * 8);
      if constexpr (KB == 1) mw >>= 32 * (u % STEPS);
      mw >>= 4 * g;
      if constexpr (KB == 2) mask_scores(sacc[0], sacc[1], mw);
      else mask_scores(sacc[0], (unsigned)mw);
    }
    // K^T fragments of the second product, read under the exponentials below
    uintx4 fkt[2 * KB][DB];
#pragma unroll
    for (int ts = 0; ts < 2 * KB; ++ts)
#pragma unroll
      for (int db = 0; db < DB; ++db) fkt[ts][db] = frag_cols<D, BF16 && !PB>(kt, db, ts, lane);
    __builtin_amdgcn_sched_barrier(0);
    // dS^T = P^T * (dP^T - delta), this lane's query; packed as operand slices of 16 keys
    uintx4 dsf[2 * KB];
#pragma unroll
    for (int ts = 0; ts < 2 * KB; ++ts)
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int kb = ts >> 1, i = 8 * (ts & 1) + 2 * jj;
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][i], qk_scale, -lse2));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][i + 1], qk_scale, -lse2));
        dsf[ts][jj] = pack2<PB>(p0 * (dpacc[kb][i] - dlt), p1 * (dpacc[kb][i + 1] - dlt));
      }
#pragma unroll
    for (int ts = 0; ts < 2 * KB; ++ts)
#pragma unroll
      for (int db = 0; db < DB; ++db)
        dqacc[db] = mfma_qk<PB>(fkt[ts][db], dsf[ts], dqacc[db]);       // dQ^T += K^T dS^T
  }

  if (prm.split > 1) {   // unscaled fp32 part; sum_parts_kernel adds the parts up
    float* part = prm.part_dq + ((int64_t)chunk * prm.B * prm.H + bh) * prm.N * D;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
        store_out4<BF16>(part, qrow * D + 32 * db + 8 * i4 + 4 * g, true, dqacc[db][4 * i4], dqacc[db][4 * i4 + 1],
                         dqacc[db][4 * i4 + 2], dqacc[db][4 * i4 + 3]);
    return;
  }
  // dQ rows leave through this wavefront's stage of the (now idle) tile buffers
  static_assert(rows_out_bytes(D, true) <= C::STAGE_BYTES, "a stage holds a wavefront's 32 result rows");
  __syncthreads();           // the other wavefront has left its last step
  const float sc = prm.sm_scale;
  rows_out<BF16, D>(lds + wv * C::STAGE_BYTES, prm.dq, b * prm.dqs[0] + h * prm.dqs[1] + ((int64_t)m * 64 + 32 * wv) * prm.dqs[2],
                    prm.dqs[2], prm.out_f32, lane, [&](int db, int i) { return dqacc[db][i] * sc; });
}

// ---------------------------------------------------------------------------------------
// dK, dV: workgroup = column block n, wavefront wv owns keys 64n + 32wv + ln
// ---------------------------------------------------------------------------------------
// QB: 32-query blocks of a tile handled per step (2: a whole tile; 1: a tile in two halves, which
// halves the fragments in flight).
// DH: -1, or at D = 256 the half (0 / 1) of the head dimension whose dK and dV columns this launch
// accumulates and writes (the first products always contract over the whole head dimension): with
// 128 columns at a time the accumulators and K, V of 32 keys are 256 registers instead of 384.
template <int D, bool BF16, bool EW, bool PB, int QB, int DH>
__global__ __launch_bounds__(128, (QB == 1 && D == 64) ? 2 : 1) void dkdv_kernel(const BwdParams prm) {
  using C = BwdCfg<D, EW, 32 * QB>;
  constexpr int KS = D / 16, STEPS = 2 / QB;
  constexpr int DB = DH < 0 ? D / 32 : D / 64, DB0 = DH < 0 ? 0 : DH * DB;   // 32-column blocks of this launch, the first one
  constexpr int PORTIONS = D == 256 ? 2 : 1, KSP = KS / PORTIONS;            // fragments of the first products in portions
  static_assert(QB == 1 || PORTIONS == 1, "whole tiles per step only without portions");
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ln = lane & 31, g = lane >> 5;
  const int nb = prm.nb;
  int bh, n;                                  // early columns of block-causal masks are the long ones
  const int per_chunk = gridDim.x / prm.split;
  const int chunk = blockIdx.x / per_chunk;
  head_and_block(blockIdx.x - chunk * per_chunk, prm.B * prm.H, nb, bh, n);
  if (n >= nb) return;
  const int b = bh / prm.H, h = bh % prm.H;
  const int mh = (prm.Bm > 1 ? b : 0) * prm.Hm + (prm.Hm > 1 ? h : 0);
  const cint_ptr_t cp = (cint_ptr_t)(uintptr_t)(prm.col_ptr + (int64_t)mh * nb);
  const cint_ptr_t rows = (cint_ptr_t)(uintptr_t)prm.row_idx;
  int u0, u1;                                                  // steps: tile u / STEPS, part u % STEPS
  {
    const int t0 = cp[n], len = cp[n + 1] - t0;                // this workgroup's share of the column's list
    u0 = (t0 + (int)((int64_t)len * chunk / prm.split)) * STEPS;
    u1 = (t0 + (int)((int64_t)len * (chunk + 1) / prm.split)) * STEPS;
  }
  const unsigned lds_addr = (unsigned)(uintptr_t)(lds_ptr_t)lds;

  const unsigned short* qg = (const unsigned short*)prm.q + b * prm.qs[0] + h * prm.qs[1];
  const unsigned short* gg = (const unsigned short*)prm.d_o + b * prm.dos[0] + h * prm.dos[1];
  const float* lse_h = prm.lse + (int64_t)bh * prm.N;
  const float* dlt_h = prm.delta + (int64_t)bh * prm.N;
  auto issue = [&](int u, int stage) {
    const int t = u / STEPS;
    const int rb = rows[t];
    const int64_t row0 = (int64_t)rb * 64 + (u % STEPS) * 32 * QB;
    const unsigned sa = lds_addr + stage * C::STAGE_BYTES;
    half_tile_load_async<D, 32 * QB>(qg + row0 * prm.qs[2], prm.qs[2], wv, lane, sa);
    half_tile_load_async<D, 32 * QB>(gg + row0 * prm.dos[2], prm.dos[2], wv, lane, sa + C::TILE_BYTES);
    stat_load_async((wv == 0 ? lse_h : dlt_h) + rb * 64, lane, sa + 2 * C::TILE_BYTES + wv * 256);   // all 64 rows of the tile
    if constexpr (EW)   // the tile's 64 mask words (one per key, bit = query), 256 bytes per wavefront
      stat_load_async(reinterpret_cast<const float*>(prm.bits_cols + (int64_t)t * 64) + wv * 64, lane,
                      sa + 2 * C::TILE_BYTES + C::STAT_BYTES + wv * 256);
  };
  if (u0 < u1) issue(u0, 0);

  const int64_t krow = (int64_t)n * 64 + 32 * wv + ln;
  const unsigned short* kp = (const unsigned short*)prm.k + b * prm.ks[0] + h * prm.ks[1] + krow * prm.ks[2];
  const unsigned short* vp = (const unsigned short*)prm.v + b * prm.vs[0] + h * prm.vs[1] + krow * prm.vs[2];
  uintx4 kfr[KS], vfr[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    kfr[s] = *reinterpret_cast<const uintx4*>(kp + 16 * s + 8 * g);
    vfr[s] = *reinterpret_cast<const uintx4*>(vp + 16 * s + 8 * g);
  }
#pragma unroll
  for (int s = 0; s < KS; ++s) { settle(kfr[s]); settle(vfr[s]); }   // no vector-memory waits in the loop, as in dq_kernel
  const float qk_scale = prm.qk_scale;

  floatx16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) { dkacc[db] = zero16(); dvacc[db] = zero16(); }

  for (int u = u0; u < u1; ++u) {
    const int stage = (u - u0) & 1;
    wait_vm<0>();
    __syncthreads();
    if (u + 1 < u1) issue(u + 1, stage ^ 1);
    const unsigned char* qt = lds + stage * C::STAGE_BYTES;
    const unsigned char* gt = qt + C::TILE_BYTES;
    const int qoff = QB == 1 ? 32 * (u % STEPS) : 0;            // first query of this step within the tile
    const float* st_lse = reinterpret_cast<const float*>(gt + C::TILE_BYTES) + qoff;
    const float* st_dlt = st_lse + 64;

    if constexpr (QB == 2) {
      // Whole tile per step, one query block after the other, so that the vector work on one query
      // block (P and dS) sits beside matrix work on the other: scores of block 0; scores of block 1
      // beside P, dS of block 0; second products of block 0 beside P, dS of block 1; second
      // products of block 1.
      floatx16 sacc[2], dpacc[2];
      uintx4 pf[4], dsf[4];
      uintx4 fq[KS], fg[KS];
      auto read_rows = [&](int qb) {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          fq[s] = frag_rows<D>(qt, 32 * qb, s, ln, g);
          fg[s] = frag_rows<D>(gt, 32 * qb, s, ln, g);
        }
      };
      auto first = [&](int qb) {
        sacc[qb] = zero16(); dpacc[qb] = zero16();
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          sacc[qb] = mfma_qk<BF16>(fq[s], kfr[s], sacc[qb]);      // S = Q K^T
          dpacc[qb] = mfma_qk<BF16>(fg[s], vfr[s], dpacc[qb]);    // dP = dO V^T
        }
      };
      unsigned long long mw = 0ull;
      if constexpr (EW)
        mw = *reinterpret_cast<const unsigned long long*>(gt + C::TILE_BYTES + C::STAT_BYTES + (32 * wv + ln) * 8) >> (4 * g);
      auto p_and_ds = [&](int qb) {          // rows of the results are queries: register i <-> query 32qb + 8(i/4) + 4g + i%4
        if constexpr (EW) mask_scores(sacc[qb], (unsigned)(mw >> (32 * qb)));
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
          for (int jh = 0; jh < 2; ++jh) {
            const int ts = 2 * qb + t2, i0 = 8 * t2 + 4 * jh;
            const int q0 = 32 * qb + 8 * (i0 >> 2) + 4 * g;
            const floatx4 l4 = *reinterpret_cast<const floatx4*>(st_lse + q0);
            const floatx4 d4 = *reinterpret_cast<const floatx4*>(st_dlt + q0);
            float p[4], ds[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float nl = EW && l4[e] == -INFINITY ? -INFINITY : -l4[e] * kLog2e;
              p[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[qb][i0 + e], qk_scale, nl));
              ds[e] = p[e] * (dpacc[qb][i0 + e] - d4[e]);
            }
            pf[ts][2 * jh] = pack2<PB>(p[0], p[1]);   pf[ts][2 * jh + 1] = pack2<PB>(p[2], p[3]);
            dsf[ts][2 * jh] = pack2<PB>(ds[0], ds[1]); dsf[ts][2 * jh + 1] = pack2<PB>(ds[2], ds[3]);
          }
      };
      uintx4 fgt[2][DB], fqt[2][DB];
      auto read_cols = [&](int qb) {
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            fgt[t2][db] = frag_cols<D, BF16 && !PB>(gt, DB0 + db, 2 * qb + t2, lane);
            fqt[t2][db] = frag_cols<D, BF16 && !PB>(qt, DB0 + db, 2 * qb + t2, lane);
          }
      };
      auto second = [&](int qb) {
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            dvacc[db] = mfma_qk<PB>(fgt[t2][db], pf[2 * qb + t2], dvacc[db]);    // dV^T += dO^T P
            dkacc[db] = mfma_qk<PB>(fqt[t2][db], dsf[2 * qb + t2], dkacc[db]);   // dK^T += Q^T dS
          }
      };
      read_rows(0);
      __builtin_amdgcn_sched_barrier(0);
      first(0);
      __builtin_amdgcn_sched_barrier(0);
      read_rows(1);
      read_cols(0);
      __builtin_amdgcn_sched_barrier(0);
      first(1);
      p_and_ds(0);
#pragma unroll
      for (int it = 0; it < 2 * KS; ++it) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      second(0);
      p_and_ds(1);
#pragma unroll
      for (int it = 0; it < 4 * DB; ++it) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      read_cols(1);
      __builtin_amdgcn_sched_barrier(0);
      second(1);
    } else {
      // operand fragments are read from LDS ahead of the block of MFMAs that consumes them
      floatx16 sacc[QB], dpacc[QB];
  #pragma unroll
      for (int qb = 0; qb < QB; ++qb) { sacc[qb] = zero16(); dpacc[qb] = zero16(); }
  #pragma unroll
      for (int pt = 0; pt < PORTIONS; ++pt) {
        uintx4 fq[QB][KSP], fg[QB][KSP];
  #pragma unroll
        for (int s = 0; s < KSP; ++s)
  #pragma unroll
          for (int qb = 0; qb < QB; ++qb) {
            fq[qb][s] = frag_rows<D>(qt, 32 * qb, pt * KSP + s, ln, g);
            fg[qb][s] = frag_rows<D>(gt, 32 * qb, pt * KSP + s, ln, g);
          }
        __builtin_amdgcn_sched_barrier(0);
  #pragma unroll
        for (int s = 0; s < KSP; ++s)
  #pragma unroll
          for (int qb = 0; qb < QB; ++qb) {
            sacc[qb] = mfma_qk<BF16>(fq[qb][s], kfr[pt * KSP + s], sacc[qb]);      // S = Q K^T
            dpacc[qb] = mfma_qk<BF16>(fg[qb][s], vfr[pt * KSP + s], dpacc[qb]);    // dP = dO V^T
          }
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (EW) {
        unsigned long long mw = *reinterpret_cast<const unsigned long long*>(
            gt + C::TILE_BYTES + C::STAT_BYTES + (32 * wv + ln) * 8);
        if constexpr (QB == 1) mw >>= qoff;
        mw >>= 4 * g;
        if constexpr (QB == 2) mask_scores(sacc[0], sacc[1], mw);
        else mask_scores(sacc[0], (unsigned)mw);
      }
      // dO^T and Q^T fragments of the second products, read under the exponentials below
      uintx4 fgt[2 * QB][DB], fqt[2 * QB][DB];
  #pragma unroll
      for (int ts = 0; ts < 2 * QB; ++ts)
  #pragma unroll
        for (int db = 0; db < DB; ++db) {
          fgt[ts][db] = frag_cols<D, BF16 && !PB>(gt, DB0 + db, ts, lane);
          fqt[ts][db] = frag_cols<D, BF16 && !PB>(qt, DB0 + db, ts, lane);
        }
      __builtin_amdgcn_sched_barrier(0);
      // rows of the results are queries: register i of block qb <-> query 32qb + 8(i/4) + 4g + i%4
      uintx4 pf[2 * QB], dsf[2 * QB];
  #pragma unroll
      for (int ts = 0; ts < 2 * QB; ++ts)
  #pragma unroll
        for (int jh = 0; jh < 2; ++jh) {
          const int qb = ts >> 1, i0 = 8 * (ts & 1) + 4 * jh;
          const int q0 = 32 * qb + 8 * (i0 >> 2) + 4 * g;
          const floatx4 l4 = *reinterpret_cast<const floatx4*>(st_lse + q0);
          const floatx4 d4 = *reinterpret_cast<const floatx4*>(st_dlt + q0);
          float p[4], ds[4];
  #pragma unroll
          for (int e = 0; e < 4; ++e) {
            // (a query without any unmasked key has lse = -inf: its P must come out as 0)
            const float nl = EW && l4[e] == -INFINITY ? -INFINITY : -l4[e] * kLog2e;
            p[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[qb][i0 + e], qk_scale, nl));
            ds[e] = p[e] * (dpacc[qb][i0 + e] - d4[e]);
          }
          pf[ts][2 * jh] = pack2<PB>(p[0], p[1]);   pf[ts][2 * jh + 1] = pack2<PB>(p[2], p[3]);
          dsf[ts][2 * jh] = pack2<PB>(ds[0], ds[1]); dsf[ts][2 * jh + 1] = pack2<PB>(ds[2], ds[3]);
        }
  #pragma unroll
      for (int ts = 0; ts < 2 * QB; ++ts)
  #pragma unroll
        for (int db = 0; db < DB; ++db) {
          dvacc[db] = mfma_qk<PB>(fgt[ts][db], pf[ts], dvacc[db]);    // dV^T += dO^T P
          dkacc[db] = mfma_qk<PB>(fqt[ts][db], dsf[ts], dkacc[db]);   // dK^T += Q^T dS
        }
  
    }
  }

  if (prm.split > 1) {   // unscaled fp32 parts; sum_parts_kernel adds them up
    const int64_t poff = ((int64_t)chunk * prm.B * prm.H + bh) * prm.N * D;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int64_t off = krow * D + 32 * (DB0 + db) + 8 * i4 + 4 * g;
        store_out4<BF16>(prm.part_dk + poff, off, true, dkacc[db][4 * i4], dkacc[db][4 * i4 + 1], dkacc[db][4 * i4 + 2],
                         dkacc[db][4 * i4 + 3]);
        store_out4<BF16>(prm.part_dv + poff, off, true, dvacc[db][4 * i4], dvacc[db][4 * i4 + 1], dvacc[db][4 * i4 + 2],
                         dvacc[db][4 * i4 + 3]);
      }
    return;
  }
  const int64_t koffh = b * prm.dks[0] + h * prm.dks[1], voffh = b * prm.dvs[0] + h * prm.dvs[1];
  void* kbase = prm.out_f32 ? (void*)((float*)prm.dk + koffh) : (void*)((unsigned short*)prm.dk + koffh);
  void* vbase = prm.out_f32 ? (void*)((float*)prm.dv + voffh) : (void*)((unsigned short*)prm.dv + voffh);
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const int col = 32 * (DB0 + db) + 8 * i4 + 4 * g;
      const int64_t off = krow * prm.dks[2] + col;
      store_out4<BF16>(kbase, off, prm.out_f32, dkacc[db][4 * i4] * prm.sm_scale, dkacc[db][4 * i4 + 1] * prm.sm_scale,
                       dkacc[db][4 * i4 + 2] * prm.sm_scale, dkacc[db][4 * i4 + 3] * prm.sm_scale);
      store_out4<BF16>(vbase, krow * prm.dvs[2] + col, prm.out_f32, dvacc[db][4 * i4], dvacc[db][4 * i4 + 1], dvacc[db][4 * i4 + 2],
                       dvacc[db][4 * i4 + 3]);
    }
}

// ---------------------------------------------------------------------------------------
// dK, dV at D = 128: workgroup = column block n, four wavefronts (one per SIMD).
// Wavefront (kh, dh) owns keys 64n + 32kh + ln and the columns 64dh .. 64dh + 63 of their dK and dV rows: half
// the accumulators of dkdv_kernel's wavefront, which, with K, V, dK and dV of its keys in 192 of 512
// registers, runs alone on its SIMD and leaves the matrix cores idle two thirds of the time.  Here a wavefront
// stays within 256 registers and two workgroups share a compute unit (two wavefronts per SIMD).
// The first products (S, dP) contract over the whole head dimension, so the two wavefronts of a key half share
// them by query block: wavefront dh computes S and dP of queries 32dh .. 32dh + 31, turns them into P and dS,
// and hands both, packed as the operand fragments of the second products, to its partner through LDS (4 KB
// each way, one barrier).  Every wavefront then runs the second products of both query blocks on its columns,
// its own block first, while the partner's P and dS are on their way.
// The per-query terms (- lse in the exponent, - delta beside dP) enter through one extra contraction slice each,
// ones x the term in three 16-bit pieces, as the forward does with its reference exponent: no vector
// instruction per element, and the row statistics need no place in LDS: a lane reads the two values of its
// query from memory a step ahead.  (Two stages of a Q and a dO tile, 64 KB, + 16 KB of exchange are exactly half
// the 160 KB of a compute unit: two workgroups per compute unit, two wavefronts per SIMD.)
// ---------------------------------------------------------------------------------------
template <int NWV, int D, int ROWS>
__device__ __forceinline__ void part_tile_load_async(const unsigned short* tile, int64_t stride, int wv, int lane,
                                                     unsigned lds_addr) {
  constexpr int CPR = D / 8, PER_WAVE = ROWS * CPR / (64 * NWV);
#pragma unroll
  for (int jj = 0; jj < PER_WAVE; ++jj) {
    const int j = wv * PER_WAVE + jj;
    const int c = j * 64 + lane, row = c / CPR, ch = c % CPR;
    const unsigned off = 2u * (unsigned)(row * (int)stride + ((ch ^ u_swz<D>(row)) * 8));
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_addr + j * 1024), "v"(off), "s"(tile) : "memory", "m0");
  }
}

// x as three 16-bit pieces (hi, mid, lo; fp16 or bf16) in the first three contraction slots of an operand slice.
// fp16 pieces hold x / PIECE_GAIN and the other operand of the slice holds PIECE_GAIN instead of ones: lse / sm_scale
// (about the largest raw q k) and delta = rowsum(O dO) (of the order |dO| sqrt(D), large under loss scaling) may lie
// far above fp16's 65504, where the first piece would be infinite and the remainders NaN.  With the gain the
// pieces reach +-4.1e6 (beyond that x is clamped: finite, wrong results instead of NaN) and are exact to
// max(2^-33 |x|, 2e-6).  bf16 pieces have fp32's range and need no gain.
constexpr float PIECE_GAIN = 64.0f;
template <bool BF16>
__device__ __forceinline__ uintx4 three_pieces(float x, bool holder) {
  unsigned short p[3];
  float rest = x;
  if constexpr (!BF16) {
    constexpr float LIM = 65000.0f;
    rest = fminf(fmaxf(x * (1.0f / PIECE_GAIN), -LIM), LIM);
  }
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    if constexpr (BF16) {
      const __bf16 v = (__bf16)rest;
      p[i] = __builtin_bit_cast(unsigned short, v);
      rest -= (float)v;
    } else {
      const _Float16 v = (_Float16)rest;
      p[i] = __builtin_bit_cast(unsigned short, v);
      rest -= (float)v;
    }
  }
  uintx4 r = {0u, 0u, 0u, 0u};
  if (holder) { r[0] = (unsigned)p[0] | ((unsigned)p[1] << 16); r[1] = (unsigned)p[2]; }
  return r;
}

constexpr int DKDV4_LDS_BYTES = 4 * 64 * 2 * 128 + 4 * 4096;   // two stages of a Q and a dO tile, 4 KB of exchange per wavefront
template <int D, bool BF16, bool PB, bool EW>
__global__ __launch_bounds__(256, 2) void dkdv4_kernel(const BwdParams prm) {
  static_assert(D == 128, "two 32-column blocks of dK and dV per wavefront");
  constexpr int KS = D / 16, DBW = D / 64;           // 32-column blocks per wavefront
  constexpr int TILE_BYTES = 64 * 2 * D, STAGE_BYTES = 2 * TILE_BYTES, EXCH_OFF = 2 * STAGE_BYTES;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kh = wv & 1, dh = wv >> 1;
  const int ln = lane & 31, g = lane >> 5;
  const int nb = prm.nb;
  int bh, n;
  const int per_chunk = gridDim.x / prm.split;
  const int chunk = blockIdx.x / per_chunk;
  head_and_block(blockIdx.x - chunk * per_chunk, prm.B * prm.H, nb, bh, n);
  if (n >= nb) return;
  const int b = bh / prm.H, h = bh % prm.H;
  const int mh = (prm.Bm > 1 ? b : 0) * prm.Hm + (prm.Hm > 1 ? h : 0);
  const cint_ptr_t cp = (cint_ptr_t)(uintptr_t)(prm.col_ptr + (int64_t)mh * nb);
  const cint_ptr_t rows = (cint_ptr_t)(uintptr_t)prm.row_idx;
  // The K and V rows this wavefront owns for the whole walk depend on the block index only: asked for first, they
  // travel while the list is looked up and the first tiles are requested.
  const int64_t krow = (int64_t)n * 64 + 32 * kh + ln;
  const unsigned short* kp = (const unsigned short*)prm.k + b * prm.ks[0] + h * prm.ks[1] + krow * prm.ks[2];
  const unsigned short* vp = (const unsigned short*)prm.v + b * prm.vs[0] + h * prm.vs[1] + krow * prm.vs[2];
  uintx4 kfr[KS], vfr[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    kfr[s] = *reinterpret_cast<const uintx4*>(kp + 16 * s + 8 * g);
    vfr[s] = *reinterpret_cast<const uintx4*>(vp + 16 * s + 8 * g);
  }
  int u0, u1;
  {
    const int t0 = cp[n], len = cp[n + 1] - t0;                // this workgroup's share of the column's list
    u0 = t0 + (int)((int64_t)len * chunk / prm.split);
    u1 = t0 + (int)((int64_t)len * (chunk + 1) / prm.split);
  }
  const unsigned lds_addr = (unsigned)(uintptr_t)(lds_ptr_t)lds;
  const unsigned short* qg = (const unsigned short*)prm.q + b * prm.qs[0] + h * prm.qs[1];
  const unsigned short* gg = (const unsigned short*)prm.d_o + b * prm.dos[0] + h * prm.dos[1];
  const float* lse_h = prm.lse + (int64_t)bh * prm.N;
  const float* dlt_h = prm.delta + (int64_t)bh * prm.N;
  const float inv_scale = 1.0f / prm.sm_scale;
  // tile copies of step u into `stage`
  auto issue = [&](int u, int stage) {
    const int rb = rows[u];
    const unsigned sa = lds_addr + stage * STAGE_BYTES;
    part_tile_load_async<4, D, 64>(qg + (int64_t)rb * 64 * prm.qs[2], prm.qs[2], wv, lane, sa);
    part_tile_load_async<4, D, 64>(gg + (int64_t)rb * 64 * prm.dos[2], prm.dos[2], wv, lane, sa + TILE_BYTES);
  };
  // lse and delta of this lane's query (of the wavefront's query block) in step u.  Ordinary loads, asked for
  // before the step's tile copies and first used after the wait for those copies at the top of the step: the
  // wait the compiler puts in front of that use then finds nothing in flight.
  // Elementwise masks: entry u of the column lists has 64 words, one per key of the tile, bit = query; a lane
  // reads the word of its key the same way.
  float st_lse = 0.f, st_dlt = 0.f;
  unsigned long long st_bits = 0ull;
  auto ask_stats = [&](int u) {
    const int q = rows[u] * 64 + 32 * dh + ln;
    st_lse = lse_h[q];
    st_dlt = dlt_h[q];
    if constexpr (EW) st_bits = prm.bits_cols[(int64_t)u * 64 + 32 * kh + ln];
  };
  if (u0 < u1) { ask_stats(u0); issue(u0, 0); }

#pragma unroll
  for (int s = 0; s < KS; ++s) { settle(kfr[s]); settle(vfr[s]); }   // K and V are there: no waits for them in the loop
  const float qk_scale = prm.qk_scale;
  // ones in the three slots the pieces occupy (second operand of the extra slices)
  const unsigned one16 = BF16 ? 0x3f80u : 0x5400u;      // 1.0 (bf16) or PIECE_GAIN = 64.0 (fp16), see three_pieces
  static_assert(PIECE_GAIN == 64.0f, "0x5400 is 64.0 in fp16");
  const uintx4 ones_frag = {g == 0 ? (one16 | (one16 << 16)) : 0u, g == 0 ? one16 : 0u, 0u, 0u};

  floatx16 dkacc[DBW], dvacc[DBW];
#pragma unroll
  for (int db = 0; db < DBW; ++db) { dkacc[db] = zero16(); dvacc[db] = zero16(); }
  uintx4* exch_mine = reinterpret_cast<uintx4*>(lds + EXCH_OFF + wv * 4096);
  const uintx4* exch_partner = reinterpret_cast<const uintx4*>(lds + EXCH_OFF + (wv ^ 2) * 4096);
  // one block of second products, the 32 queries of block qb against this wavefront's columns, in two parts: the
  // transposed fragments of dO and Q are read from LDS well ahead of the MFMAs that consume them
  auto read_cols = [&](const unsigned char* qt, const unsigned char* gt, int qb, uintx4 (&fgt)[2][DBW], uintx4 (&fqt)[2][DBW]) {
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int db = 0; db < DBW; ++db) {
        fgt[t2][db] = frag_cols<D, BF16 && !PB>(gt, DBW * dh + db, 2 * qb + t2, lane);
        fqt[t2][db] = frag_cols<D, BF16 && !PB>(qt, DBW * dh + db, 2 * qb + t2, lane);
      }
  };
  auto second = [&](const uintx4 (&fgt)[2][DBW], const uintx4 (&fqt)[2][DBW], const uintx4 (&pf)[2], const uintx4 (&dsf)[2]) {
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int db = 0; db < DBW; ++db) {
        dvacc[db] = mfma_qk<PB>(fgt[t2][db], pf[t2], dvacc[db]);    // dV^T += dO^T P
        dkacc[db] = mfma_qk<PB>(fqt[t2][db], dsf[t2], dkacc[db]);   // dK^T += Q^T dS
      }
  };

  for (int u = u0; u < u1; ++u) {
    const int stage = (u - u0) & 1;
    wait_vm<0>();
    __syncthreads();                 // the step's tiles are complete; everybody has left the previous step
    // the extra slices of this step from the statistics asked for a step ago; then the next step's
    // (a query without any unmasked key has lse = -inf; all its scores are masked below, whatever the slice holds)
    const uintx4 lse_slice = three_pieces<BF16>(EW && st_lse == -INFINITY ? 0.f : -st_lse * inv_scale, g == 0);
    const uintx4 dlt_slice = three_pieces<BF16>(-st_dlt, g == 0);
    // the mask bits of this lane's key for the queries of this wavefront's block, shifted so that bit
    // 8(i/4) + i%4 belongs to register i
    const unsigned mw = EW ? (unsigned)(st_bits >> (32 * dh)) >> (4 * g) : 0u;
    __builtin_amdgcn_sched_barrier(0);
    if (u + 1 < u1) { ask_stats(u + 1); issue(u + 1, stage ^ 1); }
    const unsigned char* qt = lds + stage * STAGE_BYTES;
    const unsigned char* gt = qt + TILE_BYTES;

    // ---- first products of this wavefront's query block: S' = Q K^T - lse / sm_scale, dP' = dO V^T - delta ----
    floatx16 sacc = zero16(), dpacc = zero16();
    {
      // (the fragments in two portions: all sixteen at once do not fit beside K, V and the accumulators)
#pragma unroll
      for (int pt = 0; pt < 2; ++pt) {
        uintx4 fq[KS / 2], fg[KS / 2];
#pragma unroll
        for (int s = 0; s < KS / 2; ++s) {
          fq[s] = frag_rows<D>(qt, 32 * dh, pt * (KS / 2) + s, ln, g);
          fg[s] = frag_rows<D>(gt, 32 * dh, pt * (KS / 2) + s, ln, g);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KS / 2; ++s) {
          sacc = mfma_qk<BF16>(fq[s], kfr[pt * (KS / 2) + s], sacc);
          dpacc = mfma_qk<BF16>(fg[s], vfr[pt * (KS / 2) + s], dpacc);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      sacc = mfma_qk<BF16>(lse_slice, ones_frag, sacc);
      dpacc = mfma_qk<BF16>(dlt_slice, ones_frag, dpacc);
    }
    if constexpr (EW) mask_scores(sacc, mw);
    // (the fragments of the own block's second products are on their way while the vector ALU works)
    uintx4 fgt_own[2][DBW], fqt_own[2][DBW];
    read_cols(qt, gt, dh, fgt_own, fqt_own);
    __builtin_amdgcn_sched_barrier(0);
    // ---- P and dS (rows of the results are queries: register i <-> query 32dh + 8(i/4) + 4g + i%4), packed as
    // the operand slices of the second products, and handed to the partner ----
    uintx4 pm[2], dm[2];             // [16-query slice of this wavefront's query block]
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
#pragma unroll
      for (int jh = 0; jh < 2; ++jh) {
        const int i0 = 8 * t2 + 4 * jh;
        float p[4], ds[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          p[e] = __builtin_amdgcn_exp2f(sacc[i0 + e] * qk_scale);
          ds[e] = p[e] * dpacc[i0 + e];
        }
        pm[t2][2 * jh] = pack2<PB>(p[0], p[1]);   pm[t2][2 * jh + 1] = pack2<PB>(p[2], p[3]);
        dm[t2][2 * jh] = pack2<PB>(ds[0], ds[1]); dm[t2][2 * jh + 1] = pack2<PB>(ds[2], ds[3]);
      }
    }
    // ---- exchange, the second products of the own query block in between ----
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) { exch_mine[(2 * t2) * 64 + lane] = pm[t2]; exch_mine[(2 * t2 + 1) * 64 + lane] = dm[t2]; }
    uintx4 fgt_oth[2][DBW], fqt_oth[2][DBW];
    read_cols(qt, gt, 1 - dh, fgt_oth, fqt_oth);
    __builtin_amdgcn_sched_barrier(0);
    second(fgt_own, fqt_own, pm, dm);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    uintx4 pp[2], dp[2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) { pp[t2] = exch_partner[(2 * t2) * 64 + lane]; dp[t2] = exch_partner[(2 * t2 + 1) * 64 + lane]; }
    second(fgt_oth, fqt_oth, pp, dp);
  }

  if (prm.split > 1) {   // unscaled fp32 parts; sum_parts_kernel adds them up
    const int64_t poff = ((int64_t)chunk * prm.B * prm.H + bh) * prm.N * D;
#pragma unroll
    for (int db = 0; db < DBW; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int64_t off = krow * D + 32 * (DBW * dh + db) + 8 * i4 + 4 * g;
        store_out4<BF16>(prm.part_dk + poff, off, true, dkacc[db][4 * i4], dkacc[db][4 * i4 + 1], dkacc[db][4 * i4 + 2],
                         dkacc[db][4 * i4 + 3]);
        store_out4<BF16>(prm.part_dv + poff, off, true, dvacc[db][4 * i4], dvacc[db][4 * i4 + 1], dvacc[db][4 * i4 + 2],
                         dvacc[db][4 * i4 + 3]);
      }
    return;
  }
  // the wavefront's 32 x 64 blocks of dK and dV leave through a stretch of the (now idle) tile stages and exchange area
  constexpr int OUT_BYTES = rows_out_bytes(32 * DBW, true);
  static_assert(4 * 2 * OUT_BYTES <= DKDV4_LDS_BYTES, "room for dK and dV of four wavefronts");
  __syncthreads();           // everybody has left the last step
  // (the lane index as a value the compiler cannot trace back: the per-lane addresses of the stores below would
  // otherwise be computed before the walk and held, or spilled, through it)
  int lane_out = lane;
  asm volatile("" : "+v"(lane_out));
  unsigned char* mine = lds + wv * 2 * OUT_BYTES;
  const int64_t r0 = (int64_t)n * 64 + 32 * kh;
  const float sc = prm.sm_scale;
  rows_out<BF16, 32 * DBW>(mine, prm.dk, b * prm.dks[0] + h * prm.dks[1] + r0 * prm.dks[2] + 32 * DBW * dh, prm.dks[2],
                           prm.out_f32, lane_out, [&](int db, int i) { return dkacc[db][i] * sc; });
  rows_out<BF16, 32 * DBW>(mine + OUT_BYTES, prm.dv, b * prm.dvs[0] + h * prm.dvs[1] + r0 * prm.dvs[2] + 32 * DBW * dh, prm.dvs[2],
                           prm.out_f32, lane_out, [&](int db, int i) { return dvacc[db][i]; });
}

// ---------------------------------------------------------------------------------------
// split > 1: out = scale * sum of the fp32 parts, rounded to the result type.  blockIdx.y: 0 dQ, 1 dK, 2 dV.
// ---------------------------------------------------------------------------------------
template <bool BF16>
__global__ __launch_bounds__(256) void sum_parts_kernel(const BwdParams prm, int64_t quads, int D) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;     // one thread per 4 consecutive values
  if (i >= quads) return;
  const float* part = blockIdx.y == 0 ? prm.part_dq : (blockIdx.y == 1 ? prm.part_dk : prm.part_dv);
  void* out = blockIdx.y == 0 ? prm.dq : (blockIdx.y == 1 ? prm.dk : prm.dv);
  const int64_t* st = blockIdx.y == 0 ? prm.dqs : (blockIdx.y == 1 ? prm.dks : prm.dvs);
  const float scale = blockIdx.y == 2 ? 1.0f : prm.sm_scale;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int c = 0; c < prm.split; ++c) acc += reinterpret_cast<const floatx4*>(part)[c * quads + i];
  // the parts are [B*H][N][D] without gaps; the result has its own strides
  const int qpr = D / 4;                                   // quads per row
  const int64_t row_all = i / qpr;
  const int col = (int)(i - row_all * qpr) * 4;
  const int bh = (int)(row_all / prm.N), row = (int)(row_all - (int64_t)bh * prm.N);
  const int b = bh / prm.H, h = bh - b * prm.H;
  store_out4<BF16>(out, b * st[0] + h * st[1] + row * st[2] + col, prm.out_f32, acc[0] * scale, acc[1] * scale,
                   acc[2] * scale, acc[3] * scale);
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
// Workgroups per row / column list.  One is enough when the launch has at least four workgroups
// per compute unit; a single long head would otherwise walk its lists on a fraction of the GPU.
static int bwd_split(int B, int H, int N) {
  const int64_t lists = (int64_t)B * H * (N / 64), want = 4 * (int64_t)compute_units();
  if (lists >= want) return 1;
  int64_t s = (want + lists - 1) / lists;
  const int cap = N / 64 / 8 > 1 ? N / 64 / 8 : 1;        // a share should have a few tiles even in a dense list
  if (s > cap) s = cap;
  return (int)(s > 8 ? 8 : s);
}

size_t bwd_workspace_bytes(int B, int H, int N, int D) {
  const size_t delta = (size_t)B * H * N * sizeof(float);
  const int split = bwd_split(B, H, N);
  return delta + (split > 1 ? (size_t)3 * split * B * H * N * D * sizeof(float) : 0);   // + parts of dQ, dK, dV
}

template <int D, bool BF16, bool EW, bool PB>
static void launch_bwd_t(const BwdParams& prm, hipStream_t st) {
  using C = BwdCfg<D, EW>;
  constexpr int KB = D >= 128 ? 1 : 2;          // dq_kernel walks D >= 128 tiles in two halves (no gain at D = 64: two wavefronts per SIMD anyway)
  using CQ = BwdCfg<D, EW, 32 * KB>;
  // dkdv_kernel (D = 64 and 256; D = 128 runs dkdv4_kernel): halves at D = 64 (191 instead of 318 registers: two
  // wavefronts per SIMD; B*H = 32 N = 8192 dense block-causal backward 1417 -> 1167 us); at D = 256 halves too, and
  // the head dimension of dK, dV in two launches.
  constexpr int QB = 1;
  using CK = BwdCfg<D, EW, 32 * QB>;
  static std::atomic<unsigned long long> configured{0};   // raising the dynamic LDS limit is idempotent
  once_per_device(configured, [] {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&dq_kernel<D, BF16, EW, PB, KB>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, CQ::LDS_BYTES);
    if constexpr (D == 256) {
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&dkdv_kernel<D, BF16, EW, PB, QB, 0>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, CK::LDS_BYTES);
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&dkdv_kernel<D, BF16, EW, PB, QB, 1>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, CK::LDS_BYTES);
    } else if constexpr (D == 128) {
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&dkdv4_kernel<D, BF16, PB, EW>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, DKDV4_LDS_BYTES);
    } else {
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&dkdv_kernel<D, BF16, EW, PB, QB, -1>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, CK::LDS_BYTES);
    }
  });
  const int BH = prm.B * prm.H;
  const int grid = ((BH + 7) / 8) * 8 * prm.nb * prm.split;   // heads in groups of 8, the last group padded
  hipLaunchKernelGGL((dq_kernel<D, BF16, EW, PB, KB>), dim3(grid), dim3(128), CQ::LDS_BYTES, st, prm);
  if constexpr (D == 256) {   // the two halves of the head dimension of dK, dV in two launches
    hipLaunchKernelGGL((dkdv_kernel<D, BF16, EW, PB, QB, 0>), dim3(grid), dim3(128), CK::LDS_BYTES, st, prm);
    hipLaunchKernelGGL((dkdv_kernel<D, BF16, EW, PB, QB, 1>), dim3(grid), dim3(128), CK::LDS_BYTES, st, prm);
  } else if constexpr (D == 128) {   // D = 128: four wavefronts per column block, two per SIMD
    hipLaunchKernelGGL((dkdv4_kernel<D, BF16, PB, EW>), dim3(grid), dim3(256), DKDV4_LDS_BYTES, st, prm);
  } else {
    hipLaunchKernelGGL((dkdv_kernel<D, BF16, EW, PB, QB, -1>), dim3(grid), dim3(128), CK::LDS_BYTES, st, prm);
  }
  if (prm.split > 1) {
    const int64_t quads = (int64_t)BH * prm.N * D / 4;
    hipLaunchKernelGGL((sum_parts_kernel<BF16>), dim3((unsigned)((quads + 255) / 256), 3), dim3(256), 0, st, prm, quads, D);
  }
}

int launch_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
               const float* lse, void* dq, void* dk, void* dv, const int32_t* row_ptr,
               const int32_t* col_idx, const int32_t* col_ptr, const int32_t* row_idx,
               const uint64_t* bits_rows, const uint64_t* bits_cols,
               const AttnShape& s, void* ws, hipStream_t st) {
  BwdParams prm;
  prm.q = q; prm.k = k; prm.v = v; prm.o = o; prm.d_o = d_o; prm.lse = lse; prm.delta = (float*)ws;
  prm.dq = dq; prm.dk = dk; prm.dv = dv;
  prm.row_ptr = row_ptr; prm.col_idx = col_idx; prm.col_ptr = col_ptr; prm.row_idx = row_idx;
  prm.bits_rows = (const unsigned long long*)bits_rows; prm.bits_cols = (const unsigned long long*)bits_cols;
  prm.B = s.B; prm.H = s.H; prm.N = s.N; prm.nb = s.N / 64; prm.Bm = s.Bm; prm.Hm = s.Hm;
  prm.out_f32 = s.out_dtype == BSATTN_F32;
  prm.split = bwd_split(s.B, s.H, s.N);
  {
    const size_t one = (size_t)prm.split * s.B * s.H * s.N * s.D;
    prm.part_dq = (float*)ws + (size_t)s.B * s.H * s.N;
    prm.part_dk = prm.part_dq + one;
    prm.part_dv = prm.part_dk + one;
  }
  prm.sm_scale = s.sm_scale;
  prm.qk_scale = s.sm_scale * kLog2e;
  for (int i = 0; i < 3; ++i) {
    prm.qs[i] = s.qs[i]; prm.ks[i] = s.ks[i]; prm.vs[i] = s.vs[i]; prm.os[i] = s.os[i]; prm.dos[i] = s.dos[i];
    prm.dqs[i] = s.dqs[i]; prm.dks[i] = s.dks[i]; prm.dvs[i] = s.dvs[i];
  }
  const bool bf = s.dtype == BSATTN_BF16;
  // bf16 gradients are rounded to 8 bits anyway: P and dS are then rounded to bf16 as well (what the
  // reference's forward does with P, fa2_fwd.py:189) and no tile needs converting; fp32 gradients of
  // bf16 inputs keep P and dS in fp16.
  const bool pb = bf && !prm.out_f32;
  const bool ew = bits_rows != nullptr;
  auto pick = [&](auto dc) {
    constexpr int DD = decltype(dc)::value;
    if (!ew) {
      if (!bf) launch_bwd_t<DD, false, false, false>(prm, st);
      else if (pb) launch_bwd_t<DD, true, false, true>(prm, st);
      else launch_bwd_t<DD, true, false, false>(prm, st);
    } else {   // elementwise mask
      if (!bf) launch_bwd_t<DD, false, true, false>(prm, st);
      else if (pb) launch_bwd_t<DD, true, true, true>(prm, st);
      else launch_bwd_t<DD, true, true, false>(prm, st);
    }
  };
  if (s.D == 64) pick(std::integral_constant<int, 64>{});
  else if (s.D == 128) pick(std::integral_constant<int, 128>{});
  else pick(std::integral_constant<int, 256>{});
  return launch_status();
}

}  // namespace bsattn
