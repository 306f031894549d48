// Measurement aid for the benchmark, built as a library of its own (libbsattn_probe.so): the matrix-core
// rate this GPU sustains for given operand data.  Not part of the attention library and not declared in
// its header.  The rate depends on the data: operands that toggle many bits draw more power and the
// clock drops, so the ceiling for real (random) activations is below the datasheet peak.
//
//   int probe_mfma_rate(const void* operands, int iters, float* sink, double* flops, void* stream)
//
// One workgroup of 8 wavefronts per compute unit; every wavefront issues iters x 8 MFMAs (32x32x16 fp16,
// fp32 accumulate) on four independent accumulator chains, whose operand fragments are read from
// `operands` (8192 bytes of device memory, 16-byte aligned: 64 lanes x 8 fragments x 8 fp16).  sink: 512
// floats of device memory (keeps the work alive); sink[511] receives the shader clock in GHz that the first
// wavefront saw over its loop (shader cycle counter against the 100 MHz wall clock: the clock the power
// management holds for this operand data).  *flops (host memory, may be NULL) receives the
// floating-point operations of the launch; time the launch with events on `stream` to obtain the rate.
// Returns 0, or -1 (a pointer is NULL), -5 (operands not 16-byte aligned), -7 (launch refused),
// -8 (iters outside [1, 2^20]).
//
//   int probe_mfma_softmax_mix(const void* operands, int iters, float* sink, double* flops, void* stream)
//
// The same with the vector instructions of the D = 64 forward's softmax beside the MFMAs, in the forward's
// proportion: per 36 MFMAs the numerators of 64 scores per lane, i.e. 64 v_exp_f32, 32 v_cvt_pk_f16_f32,
// 32 v_dot2c_f32_f16 (row sums) and, standing in for the forward's remaining vector work, 64 v_fma_f32
// (which here also keep the exponentials' arguments moving and bounded): 192 vector instructions, where the
// forward's loop has 202.  Everything stays in registers:
// no LDS, no memory traffic, no barriers.  What this sustains is the ceiling of the forward's instruction mix.
// Every wavefront issues iters x 9 MFMAs; arguments, sink and return values as above.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

__global__ __launch_bounds__(512) void mfma_rate_kernel(const uintx4* operands, int iters, float* sink) {
  const int lane = threadIdx.x & 63;
  uintx4 a[4], b[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) { a[c] = operands[lane * 8 + c]; b[c] = operands[lane * 8 + 4 + c]; }
  floatx16 acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[c][i] = 0.f;
  const long long c0 = __builtin_readcyclecounter(), w0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
      acc[r & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a[r & 3]),
                                                         __builtin_bit_cast(half8, b[(r >> 1) & 3]), acc[r & 3], 0, 0, 0);
  }
  const long long c1 = __builtin_readcyclecounter(), w1 = __builtin_amdgcn_s_memrealtime();
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[c][i];
  if (blockIdx.x == 0 && threadIdx.x < 511) sink[threadIdx.x] = s;
  if (blockIdx.x == 0 && threadIdx.x == 0) sink[511] = w1 > w0 ? 0.1f * (float)(c1 - c0) / (float)(w1 - w0) : 0.f;
}

typedef _Float16 half2 __attribute__((ext_vector_type(2)));

__global__ __launch_bounds__(512) void mfma_softmax_mix_kernel(const uintx4* operands, int iters, float* sink) {
  const int lane = threadIdx.x & 63;
  uintx4 a[4], b[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) { a[c] = operands[lane * 8 + c]; b[c] = operands[lane * 8 + 4 + c]; }
  floatx16 acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[c][i] = 0.f;
  // sixteen "scores" per lane in (-6, 0], taken from the operand data; c1 * P + c0 maps a numerator P in
  // (0, 1] back into that range
  float x[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const half2 h = __builtin_bit_cast(half2, a[i & 3][(i >> 2) & 3]);
    x[i] = -__builtin_fabsf((float)h[0]) - 0.25f * (float)(i & 3);
  }
  const float c1 = -2.0f - 0.03125f * (float)(lane & 31), c0 = -0.125f;
  const half2 ones = {(_Float16)1.0f, (_Float16)1.0f};
  float l = 0.f;
  const long long t0 = __builtin_readcyclecounter(), w0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 9; ++r) {
      acc[r & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a[r & 3]),
                                                         __builtin_bit_cast(half8, b[(r >> 1) & 3]), acc[r & 3], 0, 0, 0);
      if (r < 8) {     // two scores: two exponentials, one conversion of the pair, one row-sum step, two updates
        const int i = 2 * r;
        const float p0 = __builtin_amdgcn_exp2f(x[i]), p1 = __builtin_amdgcn_exp2f(x[i + 1]);
        const half2 hp = {(_Float16)p0, (_Float16)p1};
        l = __builtin_amdgcn_fdot2(hp, ones, l, false);
        x[i] = __builtin_fmaf(p1, c1, c0);
        x[i + 1] = __builtin_fmaf(p0, c1, c0);
      }
    }
  }
  const long long t1 = __builtin_readcyclecounter(), w1 = __builtin_amdgcn_s_memrealtime();
  float s = l;
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[c][i];
#pragma unroll
  for (int i = 0; i < 16; ++i) s += x[i];
  if (blockIdx.x == 0 && threadIdx.x < 511) sink[threadIdx.x] = s;
  if (blockIdx.x == 0 && threadIdx.x == 0) sink[511] = w1 > w0 ? 0.1f * (float)(t1 - t0) / (float)(w1 - w0) : 0.f;
}

static int probe_launch(bool mix, const void* operands, int iters, float* sink, double* flops, void* stream) {
  if (operands == nullptr || sink == nullptr) return -1;
  if (iters <= 0 || iters > (1 << 20)) return -8;
  if (((uintptr_t)operands & 15) != 0) return -5;
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  if (mix)
    hipLaunchKernelGGL(mfma_softmax_mix_kernel, dim3(cus), dim3(512), 0, (hipStream_t)stream, (const uintx4*)operands, iters, sink);
  else
    hipLaunchKernelGGL(mfma_rate_kernel, dim3(cus), dim3(512), 0, (hipStream_t)stream, (const uintx4*)operands, iters, sink);
  if (flops != nullptr) *flops = (double)cus * 8.0 * iters * (mix ? 9.0 : 8.0) * 2.0 * 32 * 32 * 16;
  return hipGetLastError() == hipSuccess ? 0 : -7;
}

extern "C" int probe_mfma_softmax_mix(const void* operands, int iters, float* sink, double* flops, void* stream) {
  return probe_launch(true, operands, iters, sink, flops, stream);
}

extern "C" int probe_mfma_rate(const void* operands, int iters, float* sink, double* flops, void* stream) {
  return probe_launch(false, operands, iters, sink, flops, stream);
}
