// Benchmark-only library (libringattn_probe.so), not part of the block-step ABI.
// Diagnostic: the bf16 MFMA rate this GPU sustains with nothing but matrix instructions in flight.
// The published dense peak assumes the maximum clock; under a full matrix load with operands
// that toggle like real data the clock settles lower, so the rate measured here is the ceiling
// any kernel made of v_mfma_f32_32x32x16_bf16 can approach on this board.
#include "ra_common.h"

namespace ra {

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16;
  x *= 0x85ebca6bu;
  x ^= x >> 13;
  x *= 0xc2b2ae35u;
  x ^= x >> 16;
  return x;
}

// One wave per SIMD, eight independent accumulator chains, operands fixed in registers.
// RANDOM = 1: operands uniform in [-2, 2) (different in every lane); 0: nearly constant operands.
template <int RANDOM>
__global__ __launch_bounds__(256) void mfma_rate_kernel(float* sink, int iters) {
  bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const unsigned h1 = probe_hash((threadIdx.x + blockIdx.x * 256u) * 64u + i * 8u + e), h2 = probe_hash(h1 + 12345u);
      a[i][e] = (bf16_t)(RANDOM ? ((int)(h1 & 0xffff) - 32768) / 16384.0f : 0.001f * threadIdx.x);
      b[i][e] = (bf16_t)(RANDOM ? ((int)(h2 & 0xffff) - 32768) / 16384.0f : 0.5f * e);
    }
  f32x16 acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  for (int it = 0; it < iters; it += 4) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 8; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i + j) & 3], b[i & 3], acc[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace ra

// Launches `blocks` workgroups of four waves (one per SIMD) that each issue iters x 8 independent
// v_mfma_f32_32x32x16_bf16 and nothing else; the caller times the launch and divides
// blocks * 4 * iters * 8 * 32768 FLOP by it.  `sink` receives blocks * 256 floats.  Returns 0, -1
// for bad arguments or the HIP error code of the launch.
extern "C" int ra_probe_mfma_rate(float* sink, int blocks, int iters, int random_operands, void* stream) {
  if (!sink || blocks <= 0 || blocks > 65536 || iters <= 0 || (iters % 4)) return -1;
  hipStream_t st = (hipStream_t)stream;
  if (random_operands) hipLaunchKernelGGL((ra::mfma_rate_kernel<1>), dim3(blocks), dim3(256), 0, st, sink, iters);
  else hipLaunchKernelGGL((ra::mfma_rate_kernel<0>), dim3(blocks), dim3(256), 0, st, sink, iters);
  return (int)hipGetLastError();
}
