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

// bf16 bits -> fp16 bits, 8 at a time (exact for the magnitudes attention inputs take)
__device__ __forceinline__ uintx4 bf16x8_to_f16x8(uintx4 x) {
  uintx4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float lo = __builtin_bit_cast(float, x[i] << 16);
    const float hi = __builtin_bit_cast(float, x[i] & 0xffff0000u);
    typedef _Float16 half2v __attribute__((ext_vector_type(2)));
    half2v h = {(_Float16)lo, (_Float16)hi};
    r[i] = __builtin_bit_cast(unsigned int, h);
  }
  return r;
}

template <int D, bool BF16>
__global__ __launch_bounds__(64) void fwd_kernel(const FwdParams prm) {
  constexpr int KS = D / 16;       // k-slices of the first product
  constexpr int DB = D / 32;       // 32-wide blocks of the head dimension
  constexpr int CPR = D / 8;       // 16-byte chunks per row
  constexpr int RP = 256 / (2 * D) > 0 ? 256 / (2 * D) : 1;  // rows per 256 bytes of LDS
  constexpr int ROWB = 2 * D;      // bytes per LDS row
  __shared__ __attribute__((aligned(16))) unsigned char lds_k[64 * ROWB];
  __shared__ __attribute__((aligned(16))) unsigned char lds_v[64 * ROWB];

  const int lane = threadIdx.x;
  const int ln = lane & 31, g = lane >> 5;
  const int p = blockIdx.x, bh = blockIdx.y;
  const int b = bh / prm.H, h = bh % prm.H;
  const int mh = (prm.Bm > 1 ? b : 0) * prm.Hm + (prm.Hm > 1 ? h : 0);
  const int nb = prm.nb;
  const int32_t* rp = prm.row_ptr + (int64_t)mh * nb;
  const HeadSplit hs = head_split(rp, nb, prm.P);
  if (p >= hs.Peff) return;
  const int t0 = split_begin(hs, p), t1 = split_begin(hs, p + 1);
  if (t0 >= t1) return;

  const unsigned short* qg = (const unsigned short*)prm.q + b * prm.qs[0] + h * prm.qs[1];
  const unsigned short* kg = (const unsigned short*)prm.k + b * prm.ks[0] + h * prm.ks[1];
  const unsigned short* vg = (const unsigned short*)prm.v + b * prm.vs[0] + h * prm.vs[1];
  const float qk_scale = prm.qk_scale;

  // first row block of the range: largest r with rp[r] <= t0 < rp[r+1]
  int r;
  {
    int lo = 0, hi = nb;  // invariant: rp[lo] <= t0 < rp[hi]
    while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (rp[mid] <= t0) lo = mid; else hi = mid; }
    r = lo;
  }
  int t = t0;
  bool first = true;
  while (t < t1) {
    const int rs = rp[r], re = rp[r + 1];
    if (re <= t) { ++r; continue; }
    const int seg_end = re < t1 ? re : t1;

    // ---- Q fragments (second operand of S^T = K Q^T): lane owns query ln (+32 qb) ----
    uintx4 qf[2][KS];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const unsigned short* qrow = qg + (int64_t)(r * 64 + qb * 32 + ln) * prm.qs[2];
#pragma unroll
      for (int s = 0; s < KS; ++s) qf[qb][s] = *reinterpret_cast<const uintx4*>(qrow + 16 * s + 8 * g);
    }
    floatx16 oacc[DB][2];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[db][qb][i] = 0.f;
    float m_i[2] = {-INFINITY, -INFINITY};
    float l_i[2] = {0.f, 0.f};  // per-lane partial sums (this lane's half of the keys)

    for (int ti = t; ti < seg_end; ++ti) {
      const int cb = prm.col_idx[ti];
      // ---- stage K and V tiles: global -> registers -> LDS (wave-private) ----
      wave_lds_sync();  // previous tile's reads are done
      {
        const unsigned short* kt = kg + (int64_t)cb * 64 * prm.ks[2];
        const unsigned short* vt = vg + (int64_t)cb * 64 * prm.vs[2];
        uintx4 kr[CPR], vr[CPR];
#pragma unroll
        for (int j = 0; j < CPR; ++j) {
          const int c = j * 64 + lane, row = c / CPR, ch = c % CPR;
          kr[j] = *reinterpret_cast<const uintx4*>(kt + (int64_t)row * prm.ks[2] + ch * 8);
          vr[j] = *reinterpret_cast<const uintx4*>(vt + (int64_t)row * prm.vs[2] + ch * 8);
        }
#pragma unroll
        for (int j = 0; j < CPR; ++j) {
          const int c = j * 64 + lane, row = c / CPR, ch = c % CPR;
          *reinterpret_cast<uintx4*>(lds_k + row * ROWB + ((ch ^ ((row / RP) % CPR)) * 16)) = kr[j];
          uintx4 vv = vr[j];
          if constexpr (BF16) vv = bf16x8_to_f16x8(vv);
          *reinterpret_cast<uintx4*>(lds_v + row * ROWB + ch * 16) = vv;
        }
      }
      wave_lds_sync();

      // ---- S^T[kb][qb] = K[kb] Q[qb]^T ----
      floatx16 sacc[2][2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int i = 0; i < 16; ++i) sacc[kb][qb][i] = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const int row = 32 * kb + ln;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          const int ch = 2 * s + g;
          const uintx4 a = *reinterpret_cast<const uintx4*>(lds_k + row * ROWB + ((ch ^ ((row / RP) % CPR)) * 16));
#pragma unroll
          for (int qb = 0; qb < 2; ++qb) sacc[kb][qb] = mfma_qk<BF16>(a, qf[qb][s], sacc[kb][qb]);
        }
      }

      // ---- online softmax, one query per lane ----
      uintx4 pf[4][2];  // P^T operand fragments: [16-key slice][qb]
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        float mx = sacc[0][qb][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) mx = fmaxf(mx, sacc[kb][qb][i]);
        mx = xhalf_max(mx);
        const float m_new = fmaxf(m_i[qb], mx * qk_scale);
        const float alpha = __builtin_amdgcn_exp2f(m_i[qb] - m_new);
        float rs_ = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][qb][i], qk_scale, -m_new));
            sacc[kb][qb][i] = pv;
            rs_ += pv;
          }
        l_i[qb] = l_i[qb] * alpha + rs_;
        m_i[qb] = m_new;
        if (__any(alpha != 1.0f)) {
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[db][qb][i] *= alpha;
        }
#pragma unroll
        for (int ts = 0; ts < 4; ++ts) {
          typedef _Float16 half2v __attribute__((ext_vector_type(2)));
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            const int i = 8 * (ts & 1) + 2 * jj;
            half2v hp = {(_Float16)sacc[ts >> 1][qb][i], (_Float16)sacc[ts >> 1][qb][i + 1]};
            pf[ts][qb][jj] = __builtin_bit_cast(unsigned int, hp);
          }
        }
      }

      // ---- O^T[db][qb] += V^T[db] P^T[qb]; V^T fragment gathered from row-major LDS ----
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int ts = 0; ts < 4; ++ts) {
          uintx4 a;
          const unsigned short* vb = reinterpret_cast<const unsigned short*>(lds_v) + (32 * db + ln);
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            const int j0 = 2 * jj, j1 = 2 * jj + 1;
            const int key0 = 16 * ts + 8 * (j0 >> 2) + 4 * g + (j0 & 3);
            const int key1 = 16 * ts + 8 * (j1 >> 2) + 4 * g + (j1 & 3);
            a[jj] = (unsigned int)vb[key0 * D] | ((unsigned int)vb[key1 * D] << 16);
          }
#pragma unroll
          for (int qb = 0; qb < 2; ++qb)
            oacc[db][qb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a),
                                                                 __builtin_bit_cast(half8, pf[ts][qb]),
                                                                 oacc[db][qb], 0, 0, 0);
        }
      }
    }  // tiles

    // ---- epilogue ----
    const bool full = (t == rs) && (seg_end == re);
    float lsum[2];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) lsum[qb] = l_i[qb] + __shfl_xor(l_i[qb], 32);
    if (full) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        const float inv = 1.0f / lsum[qb];
        const int64_t qrow = (int64_t)(r * 64 + qb * 32 + ln);
        if (prm.out_f32) {
          float* orow = (float*)prm.o + b * prm.os[0] + h * prm.os[1] + qrow * prm.os[2];
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
              floatx4 w = {oacc[db][qb][4 * i4] * inv, oacc[db][qb][4 * i4 + 1] * inv,
                           oacc[db][qb][4 * i4 + 2] * inv, oacc[db][qb][4 * i4 + 3] * inv};
              *reinterpret_cast<floatx4*>(orow + 32 * db + 8 * i4 + 4 * g) = w;
            }
        } else {
          unsigned short* orow = (unsigned short*)prm.o + b * prm.os[0] + h * prm.os[1] + qrow * prm.os[2];
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
              uintx2 w;
#pragma unroll
              for (int e = 0; e < 2; ++e) {
                const float x0 = oacc[db][qb][4 * i4 + 2 * e] * inv, x1 = oacc[db][qb][4 * i4 + 2 * e + 1] * inv;
                if constexpr (BF16) {
                  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
                  bf2 hv = {(__bf16)x0, (__bf16)x1};
                  w[e] = __builtin_bit_cast(unsigned int, hv);
                } else {
                  typedef _Float16 half2v __attribute__((ext_vector_type(2)));
                  half2v hv = {(_Float16)x0, (_Float16)x1};
                  w[e] = __builtin_bit_cast(unsigned int, hv);
                }
              }
              *reinterpret_cast<uintx2*>(orow + 32 * db + 8 * i4 + 4 * g) = w;
            }
        }
        if (prm.lse != nullptr && g == 0)
          prm.lse[((int64_t)bh * prm.N) + qrow] = (m_i[qb] + __builtin_amdgcn_logf(lsum[qb])) * 0.6931471805599453f;
      }
    } else {
      // partial slot: [acc index][lane] floats, then m[64], l[64]
      float* slot = prm.ws + ((((int64_t)bh * prm.P + p) * 2) + (first ? 0 : 1)) * partial_floats(D);
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
    first = false;
    t = seg_end;
    ++r;
  }
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
  const int64_t target = (int64_t)cus * 8 * 2;  // two rounds of 8 wavefronts per CU
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
