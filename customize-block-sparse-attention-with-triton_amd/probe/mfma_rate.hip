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

extern "C" int probe_mfma_rate(const void* operands, int iters, float* sink, double* flops, void* stream) {
  if (operands == nullptr || sink == nullptr) return -1;
  if (iters <= 0 || iters > (1 << 20)) return -8;
  if (((uintptr_t)operands & 15) != 0) return -5;
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  hipLaunchKernelGGL(mfma_rate_kernel, dim3(cus), dim3(512), 0, (hipStream_t)stream, (const uintx4*)operands, iters, sink);
  if (flops != nullptr) *flops = (double)cus * 8.0 * iters * 8.0 * 2.0 * 32 * 32 * 16;
  return hipGetLastError() == hipSuccess ? 0 : -7;
}
