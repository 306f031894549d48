// Measurement aid: the matrix-core rate this GPU sustains for given operand data.
// The rate depends on the data: operands that toggle many bits draw more power and the
// clock drops, so the ceiling for real (random) activations is below the datasheet peak.
#include "common.h"
#include "kernel_util.h"

namespace bsattn {

// Every wavefront runs iters x 8 MFMAs (32x32x16 fp16) on four independent accumulator
// chains; operand fragments come from `operands` (64 lanes x 8 fragments x 16 bytes).
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
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
      acc[r & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a[r & 3]),
                                                         __builtin_bit_cast(half8, b[(r >> 1) & 3]), acc[r & 3], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[c][i];
  if (blockIdx.x == 0) sink[threadIdx.x] = s;
}

int launch_mfma_rate(const void* operands, int iters, float* sink, double* flops, hipStream_t st) {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  hipLaunchKernelGGL(mfma_rate_kernel, dim3(cus), dim3(512), 0, st, (const uintx4*)operands, iters, sink);
  if (flops != nullptr) *flops = (double)cus * 8.0 * iters * 8.0 * 2.0 * 32 * 32 * 16;
  return launch_status();
}

}  // namespace bsattn
