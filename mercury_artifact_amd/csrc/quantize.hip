// Per-tensor e4m3 quantisation for the fp8 forward path of the ring step: s = amax(|x|) / 448,
// x_q = round-to-nearest-even e4m3(clamp(x / s, -448, 448)).  Not in the reference (its ring templates
// run bf16 only); the arithmetic is the same, bit for bit, as the torch expression
//   (x.float() / scale).clamp(-448, 448).to(torch.float8_e4m3fn)   with   scale = float(double(amax) / 448).
// Three launches on one stream: clear the maximum, reduce |x|, convert.  Bandwidth-bound: every input
// element is read twice (the second time mostly from the last-level cache for tensors that fit), one byte
// written per element.
#include "mhip_common.hpp"

namespace mhip {
namespace {

__global__ void clear_amax(unsigned int* amax_bits) { *amax_bits = 0u; }

template <bool BF16>
__device__ __forceinline__ void load8(const void* x, int64_t i, float (&v)[8]) {
  if (BF16) {
    const u32x4 w = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(x) + i);
#pragma unroll
    for (int j = 0; j < 4; ++j) { v[2 * j] = bf16_lo(w[j]); v[2 * j + 1] = bf16_hi(w[j]); }
  } else {
    const f32x4* p = reinterpret_cast<const f32x4*>(static_cast<const float*>(x) + i);
    const f32x4 a = p[0], b = p[1];
#pragma unroll
    for (int j = 0; j < 4; ++j) { v[j] = a[j]; v[4 + j] = b[j]; }
  }
}
template <bool BF16>
__device__ __forceinline__ float load1(const void* x, int64_t i) {
  return BF16 ? bf16_lo(static_cast<const uint16_t*>(x)[i]) : static_cast<const float*>(x)[i];
}

// |x| of non-NaN floats orders like its bit pattern, so the maximum is an integer atomic max on the bits
// (a NaN input wins the maximum and makes the scale NaN, as torch's amax does).
template <bool BF16>
__global__ __launch_bounds__(256) void amax_kernel(const void* __restrict__ x, int64_t n, unsigned int* amax_bits) {
  const int64_t stride = (int64_t)gridDim.x * 256 * 8;
  float m = 0.f;
  unsigned int nan_bits = 0u;
  for (int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += stride) {
    if (i + 8 <= n) {
      float v[8];
      load8<BF16>(x, i, v);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float a = fabsf(v[j]);
        if (a != a) nan_bits = 0x7fc00000u;
        m = fmaxf(m, a);
      }
    } else {
      for (int64_t e = i; e < n; ++e) {
        const float a = fabsf(load1<BF16>(x, e));
        if (a != a) nan_bits = 0x7fc00000u;
        m = fmaxf(m, a);
      }
    }
  }
  unsigned int bits = __builtin_bit_cast(unsigned int, m) | nan_bits;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned int other = (unsigned int)__shfl_xor((int)bits, off);
    bits = bits > other ? bits : other;
  }
  __shared__ unsigned int part[4];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = bits;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned int b = part[0];
    for (int w = 1; w < 4; ++w) b = b > part[w] ? b : part[w];
    atomicMax(amax_bits, b);
  }
}

__device__ __forceinline__ float scale_of(unsigned int amax_bits) {
  const float amax = __builtin_bit_cast(float, amax_bits);
  return amax > 0.f || amax != amax ? (float)((double)amax / 448.0) : 1.f;
}
__device__ __forceinline__ float clamp448(float y) {
  // NaN stays NaN (torch.clamp propagates it)
  return y != y ? y : fminf(fmaxf(y, -448.f), 448.f);
}

template <bool BF16>
__global__ __launch_bounds__(256) void convert_kernel(const void* __restrict__ x, int64_t n,
                                                      const unsigned int* __restrict__ amax_bits,
                                                      uint8_t* __restrict__ xq, float* __restrict__ scale_out) {
  const float s = scale_of(*amax_bits);
  if (blockIdx.x == 0 && threadIdx.x == 0) *scale_out = s;
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i >= n) return;
  if (i + 8 <= n) {
    float v[8];
    load8<BF16>(x, i, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = clamp448(v[j] / s);
    u32x2 w;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int packed = 0;
      packed = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * h], v[4 * h + 1], packed, false);
      packed = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * h + 2], v[4 * h + 3], packed, true);
      w[h] = (uint32_t)packed;
    }
    *reinterpret_cast<u32x2*>(xq + i) = w;
  } else {
    for (int64_t e = i; e < n; ++e) {
      const float y = clamp448(load1<BF16>(x, e) / s);
      const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(y, 0.f, 0, false);
      xq[e] = (uint8_t)(packed & 0xff);
    }
  }
}

}  // namespace
}  // namespace mhip

using namespace mhip;

extern "C" int mhip_quantize_e4m3(const void* x, int dtype, int64_t n, void* xq, float* scale, float* amax_ws,
                                  void* stream) {
  if (n < 0) return MHIP_EINVAL;
  if (dtype != MHIP_BF16 && dtype != MHIP_F32) return MHIP_EDTYPE;
  if (!scale || !amax_ws || (n > 0 && (!x || !xq))) return MHIP_EINVAL;
  if (n > 0 && (!aligned16(x) || (reinterpret_cast<uintptr_t>(xq) & 7u))) return MHIP_EALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  unsigned int* bits = reinterpret_cast<unsigned int*>(amax_ws);
  hipLaunchKernelGGL(clear_amax, dim3(1), dim3(1), 0, st, bits);
  const int64_t groups = (n + 7) / 8;
  const int64_t blocks = (groups + 255) / 256;
  const unsigned red_blocks = (unsigned)(blocks < 2048 ? (blocks > 0 ? blocks : 1) : 2048);
  const unsigned cvt_blocks = (unsigned)(blocks > 0 ? blocks : 1);
  if (blocks > 0x7fffffff) return MHIP_EUNSUPPORTED;
  if (dtype == MHIP_BF16) {
    hipLaunchKernelGGL(amax_kernel<true>, dim3(red_blocks), dim3(256), 0, st, x, n, bits);
    hipLaunchKernelGGL(convert_kernel<true>, dim3(cvt_blocks), dim3(256), 0, st, x, n, bits,
                       static_cast<uint8_t*>(xq), scale);
  } else {
    hipLaunchKernelGGL(amax_kernel<false>, dim3(red_blocks), dim3(256), 0, st, x, n, bits);
    hipLaunchKernelGGL(convert_kernel<false>, dim3(cvt_blocks), dim3(256), 0, st, x, n, bits,
                       static_cast<uint8_t*>(xq), scale);
  }
  return launch_status();
}
