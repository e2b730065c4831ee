// A measuring stick, not part of the attention path: a loop of nothing but 32x32x16 bf16 MFMAs on operands that stay
// in registers.  Held for seconds on N(0,1) data it shows what the socket's power limit leaves of the matrix peak
// before any softmax, LDS or HBM work (the benchmark's power report runs it beside the attention kernels).
#include "fox_common.hpp"
#include "fox_kernels.hpp"

namespace fox {

// One workgroup of four waves, one wave per SIMD when launched with one workgroup per CU.  Every wave keeps eight A
// and eight B operands (operands: 16 x 64 lanes x 16 bytes, any 16-bit pattern) and four accumulators in rotation;
// both operands change with every instruction.  32 MFMAs per iteration and wave.
__global__ __launch_bounds__(256, 1) void mfma_probe_kernel(const u32x4* __restrict__ operands, float* sink, int iters) {
  u32x4 a[8], b[8];
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = operands[i * 64 + lane];
    b[i] = operands[(8 + i) * 64 + lane];
  }
  f32x16 c[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) c[j][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int g = 0; g < 8; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) c[j] = Bf16::mfma32(a[(g + 2 * j) & 7], b[(g + 2 * j + 1) & 7], c[j]);
    if ((it & 255) == 255) {  // keep the accumulators in range
#pragma unroll
      for (int j = 0; j < 4; ++j) c[j] *= 1e-3f;
    }
  }
  float t = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) t += c[j][r];
  if (t == 12345.678f) sink[0] = t;  // never true in practice: keeps the loop alive
}

hipError_t launch_mfma_probe(const void* operands, float* sink, int workgroups, int iters, hipStream_t s) {
  hipLaunchKernelGGL(mfma_probe_kernel, dim3((unsigned)workgroups), dim3(256), 0, s, reinterpret_cast<const u32x4*>(operands), sink, iters);
  return hipGetLastError();
}

}  // namespace fox
