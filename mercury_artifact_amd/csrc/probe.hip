// Measurement aid (no counterpart in the reference): what the matrix pipes of this GPU sustain on a loop of
// nothing but v_mfma_f32_32x32x16_bf16, the instruction both contractions of the bf16 block kernels are made
// of.  The chip is power-managed: with operands that toggle every bit the clock settles well below nominal,
// so this is the ceiling the attention kernels should be read against on a given box.
#include "mhip_common.hpp"

namespace mhip {
namespace {

// One wavefront per SIMD, four independent accumulator chains, operands alternate between two register sets.
template <bool RANDOM>
__global__ __launch_bounds__(256) void mfma_ceiling_kernel(float* sink, long long* cycles, int iters) {
  bf16x8 a[2], b[2];
  uint32_t r = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      r = r * 1664525u + 1013904223u;
      a[s][i] = RANDOM ? (__bf16)(((int)(r >> 8) % 2001 - 1000) * 0.001f) : (__bf16)0.5f;
      r = r * 1664525u + 1013904223u;
      b[s][i] = RANDOM ? (__bf16)(((int)(r >> 8) % 2001 - 1000) * 0.001f) : (__bf16)0.25f;
    }
  f32x16 acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[c][j] = 0.f;
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[u & 1], b[u & 1], acc[c], 0, 0, 0);
  }
  const long long t1 = clock64();
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += acc[c][j];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
  if (threadIdx.x == 0 && blockIdx.x == 0) cycles[0] = t1 - t0;
}

}  // namespace
}  // namespace mhip

using namespace mhip;

extern "C" int mhip_probe_mfma_ceiling(float* sink, long long* cycles, int workgroups, int iters,
                                       int random_operands, void* stream) {
  if (workgroups <= 0 || iters <= 0) return MHIP_EINVAL;
  if (!sink || !cycles) return MHIP_EINVAL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (random_operands)
    hipLaunchKernelGGL(mfma_ceiling_kernel<true>, dim3(workgroups), dim3(256), 0, st, sink, cycles, iters);
  else
    hipLaunchKernelGGL(mfma_ceiling_kernel<false>, dim3(workgroups), dim3(256), 0, st, sink, cycles, iters);
  return launch_status();
}
