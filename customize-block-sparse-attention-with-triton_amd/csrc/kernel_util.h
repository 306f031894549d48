// Device-side helpers shared by the attention kernels: vector types, MFMA wrappers, LDS tile
// swizzles, asynchronous global->LDS tile copies and output stores.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

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

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// Two fp32 values rounded to the 16-bit type of the second products (PB: bf16, else fp16), packed.
template <bool PB>
__device__ __forceinline__ unsigned int pack2(float a, float b) {
  if constexpr (PB) {
    const bf16x2 h = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(unsigned int, h);
  } else {
    const half2v h = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(unsigned int, h);
  }
}

// acc + the two packed 16-bit values of x (what a second product will see of them)
template <bool PB>
__device__ __forceinline__ float add_packed2(unsigned int x, float acc) {
  if constexpr (PB) {
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, x), ones, acc, false);
  } else {
    const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, x), ones, acc, false);
  }
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
// (D = 256: the D = 128 patterns on the low four bits of the 32 chunk indices of a row)
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
#pragma unroll
  for (int j = 0; j < D / 8; ++j)
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_addr + j * 1024), "v"(off[j]), "s"(tile) : "memory", "m0");
}


// one instruction of tile_load_async: 64 x 16 bytes to lds_addr (+ lane*16)
__device__ __forceinline__ void tile_load_async_one(const unsigned short* tile, unsigned off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(lds_addr), "v"(off), "s"(tile) : "memory", "m0");
}

// Four consecutive instructions of a tile copy whose rows follow each other without gaps: the
// immediate offset of the instruction applies to the source and to the LDS address alike, so the
// four share one scalar base and one m0.
__device__ __forceinline__ void tile_load_async_four(const unsigned short* src, unsigned o0, unsigned o1, unsigned o2,
                                                     unsigned o3, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %5\n\tglobal_load_lds_dwordx4 %2, %5 offset:1024\n\t"
               "global_load_lds_dwordx4 %3, %5 offset:2048\n\tglobal_load_lds_dwordx4 %4, %5 offset:3072"
               :: "s"(lds_addr), "v"(o0), "v"(o1), "v"(o2), "v"(o3), "s"(src) : "memory", "m0");
}

template <int N> __device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
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


// The 32 result rows of a wavefront leave through LDS, so that a store instruction writes 16 bytes per lane with
// consecutive lanes along a row (whole rows, or 128-byte stretches of them) instead of 8 or 16 bytes in each of
// 32 rows.  The lane holds, of row `ln` of the 32, value(db, i) for column 32 db + 8 (i / 4) + 4 g + i % 4 (the
// layout in which a 32x32 MFMA result holds its rows), db < NCOL / 32.
// stage: ROWS_OUT_BYTES(NCOL, out_f32) bytes of LDS that only this wavefront touches (its LDS accesses are executed
// in order, so the reads below see the writes above them without a barrier).
// out + elem_off: row 0, first of the NCOL columns; row_stride in elements; rows 16-byte aligned.
__host__ __device__ constexpr int rows_out_bytes(int ncol, bool out_f32) { return 32 * (ncol * (out_f32 ? 4 : 2) + 16); }
template <bool BF16, int NCOL, typename F>
__device__ __forceinline__ void rows_out(unsigned char* stage, void* out, int64_t elem_off, int64_t row_stride,
                                         bool out_f32, int lane, F&& value) {
  const int ln = lane & 31, g = lane >> 5;
  if (out_f32) {
    constexpr int PITCH = NCOL * 4 + 16, LPR = NCOL / 4, RPI = 64 / LPR;   // lanes per row, rows per instruction
#pragma unroll
    for (int db = 0; db < NCOL / 32; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const floatx4 w = {value(db, 4 * i4), value(db, 4 * i4 + 1), value(db, 4 * i4 + 2), value(db, 4 * i4 + 3)};
        *reinterpret_cast<floatx4*>(stage + ln * PITCH + (32 * db + 8 * i4 + 4 * g) * 4) = w;
      }
    __builtin_amdgcn_wave_barrier();
    float* o = (float*)out + elem_off;
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
      const int r = it * RPI + lane / LPR, c = lane % LPR;
      const floatx4 w = *reinterpret_cast<const floatx4*>(stage + r * PITCH + 16 * c);
      *reinterpret_cast<floatx4*>(o + r * row_stride + 4 * c) = w;
    }
  } else {
    constexpr int PITCH = NCOL * 2 + 16, LPR = NCOL / 8, RPI = 64 / LPR;
#pragma unroll
    for (int db = 0; db < NCOL / 32; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const uintx2 w = {pack2<BF16>(value(db, 4 * i4), value(db, 4 * i4 + 1)), pack2<BF16>(value(db, 4 * i4 + 2), value(db, 4 * i4 + 3))};
        *reinterpret_cast<uintx2*>(stage + ln * PITCH + (32 * db + 8 * i4 + 4 * g) * 2) = w;
      }
    __builtin_amdgcn_wave_barrier();
    unsigned short* o = (unsigned short*)out + elem_off;
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
      const int r = it * RPI + lane / LPR, c = lane % LPR;
      const uintx4 w = *reinterpret_cast<const uintx4*>(stage + r * PITCH + 16 * c);
      *reinterpret_cast<uintx4*>(o + r * row_stride + 8 * c) = w;
    }
  }
}

// Partial results cross workgroups (and the L2 slices of different XCDs) inside one launch:
// they are written and read with device-scope accesses, which go to the point of coherence.
__device__ __forceinline__ void coherent_store(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float coherent_load(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// The same accesses 16 bytes wide (p 16-byte aligned), written out, since an atomic type of that size does not
// exist: `sc1` is what the compiler puts on the 4-byte ones above.
__device__ __forceinline__ void coherent_store4(float* p, float a, float b, float c, float d) {
  const floatx4 v = {a, b, c, d};
  asm volatile("global_store_dwordx4 %0, %1, off sc1" :: "v"(p), "v"(v) : "memory");
}
// Four such loads, 1 KB apart, and the wait for them (and for every earlier vector memory access of the wavefront)
// in one statement: the compiler does not count loads it did not issue, so the values must not leave the statement
// before they have arrived.
__device__ __forceinline__ void coherent_load4x4(const float* p, floatx4& a, floatx4& b, floatx4& c, floatx4& d) {
  asm volatile("global_load_dwordx4 %0, %4, off sc1\n\tglobal_load_dwordx4 %1, %4, off offset:1024 sc1\n\t"
               "global_load_dwordx4 %2, %4, off offset:2048 sc1\n\tglobal_load_dwordx4 %3, %4, off offset:3072 sc1\n\t"
               "s_waitcnt vmcnt(0)"
               : "=&v"(a), "=&v"(b), "=&v"(c), "=&v"(d) : "v"(p) : "memory");
}

// Swizzle for tiles that are read both ways (operand reads of 32 consecutive rows and
// transpose reads of 4 consecutive rows x 64 bytes): a bijection of the row bits that
// separates both access patterns over the 64 LDS banks.
template <int D> __device__ __forceinline__ int u_swz(int row) {   // (D = 256 as D = 128, on the low four chunk bits)
  if (D == 64) { const int x = (row >> 1) & 7; return ((x & 1) << 2) | (x >> 1); }
  return ((row & 3) << 2) | ((row >> 2) & 3);
}

}  // namespace bsattn
