// Shared device/host helpers for the gfx950 ring-attention step kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mercury_hip.h"

namespace mhip {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Two fp32 -> one dword of two bf16 (round to nearest even), low half = a.
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  f32x2 v = {a, b};
  bf16x2 r = __builtin_convertvector(v, bf16x2);
  return __builtin_bit_cast(uint32_t, r);
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

// max / sum of x over the lane pair (l, l ^ 32).  v_permlane32_swap exchanges the upper half of
// its first operand with the lower half of its second, so with both operands = x every lane ends
// up holding {own value, partner's value} in the two results (in an order that depends on the
// half) -- a symmetric combine needs no lane test.  The two results are taken out as ints first:
// __builtin_bit_cast applied directly to r[1] reads r[0] with this compiler.
__device__ __forceinline__ void pair_exchange(float x, float& a, float& b) {
  const int xi = __float_as_int(x);
  auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
  const int r0 = r[0], r1 = r[1];
  a = __int_as_float(r0);
  b = __int_as_float(r1);
}
__device__ __forceinline__ float pair_max(float x) {
  float a, b;
  pair_exchange(x, a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float pair_sum(float x) {
  float a, b;
  pair_exchange(x, a, b);
  return a + b;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Buffer descriptor over `bytes` bytes at `base`, as four scalar words: loads whose offset (vector +
// scalar part) falls past the end return zero.
__device__ __forceinline__ u32x4 rsrc_words(const void* base, uint32_t bytes) {
  const uint64_t a = (uint64_t)base;
  u32x4 r;
  // wavefront-uniform by construction; readfirstlane makes that visible to the register allocator
  r[0] = __builtin_amdgcn_readfirstlane((uint32_t)a);
  r[1] = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
  r[2] = __builtin_amdgcn_readfirstlane(bytes);
  r[3] = 0x00020000u;
  return r;
}

// Global -> LDS copy of 16 (or 4) bytes per lane without passing through registers: lane l's bytes land
// at LDS address `lds_addr` + 16 l (+ 4 l); the base is wavefront-uniform and travels in M0.  Lanes whose
// offset is out of the descriptor's range write zeros.  Completion is counted by vmcnt.  Written as
// inline assembly so that the compiler's own wait-count insertion does not see the copies: it would
// otherwise wait for all of them before every transposing LDS read.  The kernels place the waits by hand.
// M0 is written here and is not on the clobber list: the compiler treats it as a reserved register, warns
// that a clobber of it "may not be preserved" and ignores it.  That is safe as long as nothing else in a
// kernel that copies this way needs M0 (no register-indexed moves, no s_sendmsg, no GWS, no other LDS-direct
// load): every copy sets M0 itself immediately before its load, so it never relies on an earlier value.
__device__ __forceinline__ void copy16_to_lds(u32x4 rsrc, uint32_t lds_addr, int voffset, int soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :: "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voffset), "s"(rsrc),
                  "s"(__builtin_amdgcn_readfirstlane(soffset)) : "memory");
}
__device__ __forceinline__ void copy4_to_lds(u32x4 rsrc, uint32_t lds_addr, int voffset, int soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
               :: "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voffset), "s"(rsrc),
                  "s"(__builtin_amdgcn_readfirstlane(soffset)) : "memory");
}

// Tiles copied that way are rows of 256 bytes (128 bf16) without padding; chunk c (16 bytes) of row r is
// kept at chunk position c ^ lds_row_swizzle(r).  With this map both access patterns of the MFMA operand
// reads are free of bank conflicts: 32 consecutive rows x one chunk (ds_read_b128 of a row-major operand)
// and 8 rows x 4 consecutive chunks (ds_read_b64_tr_b16 of a transposed operand).
__device__ __forceinline__ constexpr int lds_row_swizzle(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int launch_status() {
  return hipGetLastError() == hipSuccess ? MHIP_OK : MHIP_ELAUNCH;
}

}  // namespace mhip
