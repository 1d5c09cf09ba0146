// Bandwidth-bound elementwise kernels of the ring-attention step for gfx950:
//   * LSE-rescale merge of a block result into the fp32 accumulators
//     (utils/flash_attn_dsl.py:31-71 of the reference), with the first-call cast and the final
//     bf16 / (B,H,S) epilogue (utils/flash_attn_dsl.py:178-179) available as fused variants;
//   * the packed twin flash_reduce (utils/flash_attn_dsl.py:293-305) and the pack that feeds it
//     (utils/flash_attn_dsl.py:396);
//   * fp32 gradient accumulation of bf16 block gradients (utils/attn_bwd_dsl.py:117-129).
// Every kernel moves each byte once with 16-byte accesses; the arithmetic is a handful of fp32
// operations per element and two transcendentals per row.
#include "mhip_common.hpp"

namespace mhip {
namespace {

// Weights of the merge for one row.  The reference computes
//   out' = out - sigmoid(bl - lse) * (out - bo),   lse' = lse - logsigmoid(lse - bl);
// here w = sigmoid(bl - lse) and lse' = max + log1p(exp(-|bl - lse|)), which is the same value
// without overflow; a -inf operand makes the other one the result.
__device__ __forceinline__ void merge_weights(float lse, float bl, float& w, float& new_lse) {
  if (bl == -INFINITY) { w = 0.f; new_lse = lse; return; }
  if (lse == -INFINITY) { w = 1.f; new_lse = bl; return; }
  const float d = bl - lse;
  const float e = __expf(-fabsf(d));                 // in (0, 1]
  const float inv = 1.f / (1.f + e);
  w = d >= 0.f ? inv : e * inv;                        // sigmoid(d)
  new_lse = fmaxf(lse, bl) + log1pf(e);
}

#ifndef MHIP_MERGE_NT
#define MHIP_MERGE_NT 2      // bit 0: non-temporal accumulator loads, bit 1: non-temporal accumulator stores
#endif
__device__ __forceinline__ f32x4 stream_load(const f32x4* p) {
  return (MHIP_MERGE_NT & 1) ? __builtin_nontemporal_load(p) : *p;
}
__device__ __forceinline__ void stream_store(f32x4 v, f32x4* p) {
  if (MHIP_MERGE_NT & 2) __builtin_nontemporal_store(v, p); else *p = v;
}

struct MergeParams {
  const float* acc_out; const float* acc_lse;
  const uint16_t* block_out; const float* block_lse;
  float* dst_out; float* dst_lse;
  uint16_t* final_out; float* final_lse;
  int B, Sq, Hq;
  int64_t rows;
  int64_t ao_sb, ao_ss, ao_sh, al_sb, al_ss, al_sh, bo_sb, bo_ss, bo_sh, bl_sb, bl_sh;
  int64_t do_sb, do_ss, do_sh, dl_sb, dl_ss, dl_sh;
};

// One row = LPR lanes x 4 contiguous head-dim values, ROWS rows per thread.  Measured on MI355X at
// 131072 rows x 128: two rows per thread with non-temporal stores is the fastest setting (5.8 TB/s in
// place, 5.2 TB/s into a separate destination); more rows per thread or non-temporal loads are slower.
template <int LPR, int ROWS, bool FIRST, bool FINAL>
__global__ __launch_bounds__(256) void lse_merge_kernel(const MergeParams p) {
  constexpr int D = LPR * 4;
  constexpr int kRowsPerPass = 256 / LPR;
  const int sub = threadIdx.x / LPR;
  const int col = (threadIdx.x % LPR) * 4;
  const int64_t row0 = (int64_t)blockIdx.x * (kRowsPerPass * ROWS) + sub;

  f32x4 acc[ROWS];
  u32x2 blk[ROWS];
  float lse[ROWS], bl[ROWS];
  int64_t o_off[ROWS], l_off[ROWS], f_off[ROWS];
  bool live[ROWS];
  // (b, s, h) of the first row by division (row counts fit 32 bits: checked on the host), of the
  // following rows by stepping
  const uint32_t first = row0 < p.rows ? (uint32_t)row0 : 0u;
  uint32_t h = first % (uint32_t)p.Hq;
  const uint32_t bs0 = first / (uint32_t)p.Hq;
  uint32_t s = bs0 % (uint32_t)p.Sq;
  uint32_t b = bs0 / (uint32_t)p.Sq;
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int64_t row = row0 + (int64_t)r * kRowsPerPass;
    live[r] = row < p.rows;
    if (r > 0) {
      h += kRowsPerPass;
      while (h >= (uint32_t)p.Hq) {
        h -= (uint32_t)p.Hq;
        if (++s == (uint32_t)p.Sq) { s = 0; ++b; }
      }
    }
    o_off[r] = b * p.do_sb + s * p.do_ss + h * p.do_sh + col;
    l_off[r] = b * p.dl_sb + s * p.dl_ss + h * p.dl_sh;
    f_off[r] = ((int64_t)b * p.Hq + h) * p.Sq + s;
    if (live[r]) {
      blk[r] = *reinterpret_cast<const u32x2*>(p.block_out + b * p.bo_sb + s * p.bo_ss + h * p.bo_sh + col);
      bl[r] = p.block_lse[b * p.bl_sb + h * p.bl_sh + s];
      if (!FIRST) {
        acc[r] = stream_load(reinterpret_cast<const f32x4*>(p.acc_out + b * p.ao_sb + s * p.ao_ss + h * p.ao_sh + col));
        lse[r] = p.acc_lse[b * p.al_sb + s * p.al_ss + h * p.al_sh];
      }
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    if (!live[r]) continue;
    f32x4 bo;
    bo[0] = bf16_lo(blk[r][0]); bo[1] = bf16_hi(blk[r][0]);
    bo[2] = bf16_lo(blk[r][1]); bo[3] = bf16_hi(blk[r][1]);
    f32x4 res;
    float new_lse;
    if (FIRST) {
      res = bo;
      new_lse = bl[r];
    } else {
      float w;
      merge_weights(lse[r], bl[r], w, new_lse);
#pragma unroll
      for (int j = 0; j < 4; ++j) res[j] = acc[r][j] - w * (acc[r][j] - bo[j]);
    }
    if (p.dst_out != nullptr) {
      stream_store(res, reinterpret_cast<f32x4*>(p.dst_out + o_off[r]));
      if (col == 0) p.dst_lse[l_off[r]] = new_lse;
    }
    if (FINAL) {
      u32x2 w2;
      w2[0] = pack_bf16(res[0], res[1]);
      w2[1] = pack_bf16(res[2], res[3]);
      const int64_t row = row0 + (int64_t)r * kRowsPerPass;
      *reinterpret_cast<u32x2*>(p.final_out + row * D + col) = w2;
      if (col == 0) p.final_lse[f_off[r]] = new_lse;
    }
  }
}

// Generic head dimension: one thread per (row, 4-element group) is replaced by one thread per
// element; used only when D is not 32 / 64 / 128 / 256.
template <bool FIRST, bool FINAL>
__global__ __launch_bounds__(256) void lse_merge_generic(const MergeParams p, int D) {
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= p.rows * D) return;
  const int64_t row = e / D;
  const int col = (int)(e % D);
  const int h = (int)(row % p.Hq);
  const int64_t bs = row / p.Hq;
  const int s = (int)(bs % p.Sq);
  const int b = (int)(bs / p.Sq);
  const float bo = bf16_lo(p.block_out[b * p.bo_sb + s * p.bo_ss + h * p.bo_sh + col]);
  const float bl = p.block_lse[b * p.bl_sb + h * p.bl_sh + s];
  float res = bo, new_lse = bl;
  if (!FIRST) {
    const float a = p.acc_out[b * p.ao_sb + s * p.ao_ss + h * p.ao_sh + col];
    float w;
    merge_weights(p.acc_lse[b * p.al_sb + s * p.al_ss + h * p.al_sh], bl, w, new_lse);
    res = a - w * (a - bo);
  }
  if (p.dst_out != nullptr) {
    p.dst_out[b * p.do_sb + s * p.do_ss + h * p.do_sh + col] = res;
    if (col == 0) p.dst_lse[b * p.dl_sb + s * p.dl_ss + h * p.dl_sh] = new_lse;
  }
  if (FINAL) {
    p.final_out[row * D + col] = (uint16_t)(pack_bf16(res, 0.f) & 0xffffu);
    if (col == 0) p.final_lse[((int64_t)b * p.Hq + h) * p.Sq + s] = new_lse;
  }
}

template <int LPR>
void launch_merge(const MergeParams& p, bool first, bool fin, hipStream_t st) {
  #ifndef MHIP_MERGE_ROWS
#define MHIP_MERGE_ROWS 2
#endif
  constexpr int ROWS = MHIP_MERGE_ROWS;
  constexpr int kRowsPerBlock = (256 / LPR) * ROWS;
  const dim3 grid((unsigned)((p.rows + kRowsPerBlock - 1) / kRowsPerBlock)), block(256);
  if (first && fin) hipLaunchKernelGGL((lse_merge_kernel<LPR, ROWS, true, true>), grid, block, 0, st, p);
  else if (first) hipLaunchKernelGGL((lse_merge_kernel<LPR, ROWS, true, false>), grid, block, 0, st, p);
  else if (fin) hipLaunchKernelGGL((lse_merge_kernel<LPR, ROWS, false, true>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((lse_merge_kernel<LPR, ROWS, false, false>), grid, block, 0, st, p);
}

// The same merge with eight head-dim values per lane: one 16-byte load of the bf16 block row piece, two
// 16-byte loads and stores of the fp32 accumulator.  Measured at 131072 rows x 128 against the kernel
// above: 29.1 vs 30.5 us into a separate destination, 28.0 vs 29.2 us in place, 21.9 vs 29.8 us with the
// fused bf16 epilogue; the first-call cast is faster with four values per lane (16.8 vs 21.1 us) and stays
// there.  One row per thread is the fastest setting here.
#ifndef MHIP_MERGE8_ROWS
#define MHIP_MERGE8_ROWS 1
#endif
template <int LPR, int ROWS, bool FIRST, bool FINAL>
__global__ __launch_bounds__(256) void lse_merge_kernel8(const MergeParams p) {
  constexpr int D = LPR * 8;
  constexpr int kRowsPerPass = 256 / LPR;
  const int sub = threadIdx.x / LPR;
  const int col = (threadIdx.x % LPR) * 8;
  const int64_t row0 = (int64_t)blockIdx.x * (kRowsPerPass * ROWS) + sub;
  f32x4 acc[ROWS][2];
  u32x4 blk[ROWS];
  float lse[ROWS], bl[ROWS];
  int64_t o_off[ROWS], l_off[ROWS], f_off[ROWS];
  bool live[ROWS];
  const uint32_t first = row0 < p.rows ? (uint32_t)row0 : 0u;
  uint32_t h = first % (uint32_t)p.Hq;
  const uint32_t bs0 = first / (uint32_t)p.Hq;
  uint32_t s = bs0 % (uint32_t)p.Sq;
  uint32_t b = bs0 / (uint32_t)p.Sq;
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int64_t row = row0 + (int64_t)r * kRowsPerPass;
    live[r] = row < p.rows;
    if (r > 0) {
      h += kRowsPerPass;
      while (h >= (uint32_t)p.Hq) {
        h -= (uint32_t)p.Hq;
        if (++s == (uint32_t)p.Sq) { s = 0; ++b; }
      }
    }
    o_off[r] = b * p.do_sb + s * p.do_ss + h * p.do_sh + col;
    l_off[r] = b * p.dl_sb + s * p.dl_ss + h * p.dl_sh;
    f_off[r] = ((int64_t)b * p.Hq + h) * p.Sq + s;
    if (live[r]) {
      blk[r] = *reinterpret_cast<const u32x4*>(p.block_out + b * p.bo_sb + s * p.bo_ss + h * p.bo_sh + col);
      bl[r] = p.block_lse[b * p.bl_sb + h * p.bl_sh + s];
      if (!FIRST) {
        const f32x4* ap = reinterpret_cast<const f32x4*>(p.acc_out + b * p.ao_sb + s * p.ao_ss + h * p.ao_sh + col);
        acc[r][0] = stream_load(ap);
        acc[r][1] = stream_load(ap + 1);
        lse[r] = p.acc_lse[b * p.al_sb + s * p.al_ss + h * p.al_sh];
      }
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    if (!live[r]) continue;
    float bo[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) { bo[2 * j] = bf16_lo(blk[r][j]); bo[2 * j + 1] = bf16_hi(blk[r][j]); }
    float res[8];
    float new_lse;
    if (FIRST) {
#pragma unroll
      for (int j = 0; j < 8; ++j) res[j] = bo[j];
      new_lse = bl[r];
    } else {
      float w;
      merge_weights(lse[r], bl[r], w, new_lse);
#pragma unroll
      for (int j = 0; j < 8; ++j) { const float a = acc[r][j >> 2][j & 3]; res[j] = a - w * (a - bo[j]); }
    }
    if (p.dst_out != nullptr) {
      f32x4* dp = reinterpret_cast<f32x4*>(p.dst_out + o_off[r]);
      stream_store(f32x4{res[0], res[1], res[2], res[3]}, dp);
      stream_store(f32x4{res[4], res[5], res[6], res[7]}, dp + 1);
      if (col == 0) p.dst_lse[l_off[r]] = new_lse;
    }
    if (FINAL) {
      u32x4 w4;
#pragma unroll
      for (int j = 0; j < 4; ++j) w4[j] = pack_bf16(res[2 * j], res[2 * j + 1]);
      const int64_t row = row0 + (int64_t)r * kRowsPerPass;
      *reinterpret_cast<u32x4*>(p.final_out + row * D + col) = w4;
      if (col == 0) p.final_lse[f_off[r]] = new_lse;
    }
  }
}

template <int LPR>
void launch_merge8(const MergeParams& p, bool first, bool fin, hipStream_t st) {
  constexpr int ROWS = MHIP_MERGE8_ROWS;
  constexpr int kRowsPerBlock = (256 / LPR) * ROWS;
  const dim3 grid((unsigned)((p.rows + kRowsPerBlock - 1) / kRowsPerBlock)), block(256);
  if (first && fin) hipLaunchKernelGGL((lse_merge_kernel8<LPR, ROWS, true, true>), grid, block, 0, st, p);
  else if (first) hipLaunchKernelGGL((lse_merge_kernel8<LPR, ROWS, true, false>), grid, block, 0, st, p);
  else if (fin) hipLaunchKernelGGL((lse_merge_kernel8<LPR, ROWS, false, true>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((lse_merge_kernel8<LPR, ROWS, false, false>), grid, block, 0, st, p);
}

// ---- packed form -----------------------------------------------------------------------------------
// The buffers are flat fp32 arrays of rows x (D+1); a row is 4(D+1) bytes long, which is not a
// multiple of 16 for D = 128, so the kernel walks the flat array in aligned groups of four floats
// and looks up the row (and its two LSEs) of every element.  Threads read the LSE column of rows
// whose other elements belong to other threads, so dst must not overlap lhs or rhs.
__global__ __launch_bounds__(256) void flash_reduce_kernel(const float* __restrict__ lhs,
                                                           const float* __restrict__ rhs,
                                                           float* __restrict__ dst,
                                                           int64_t total, int W) {
  const int64_t g = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (g >= total) return;
  float a[4], b[4];
  if (g + 4 <= total) {
    const f32x4 va = *reinterpret_cast<const f32x4*>(lhs + g);
    const f32x4 vb = *reinterpret_cast<const f32x4*>(rhs + g);
#pragma unroll
    for (int j = 0; j < 4; ++j) { a[j] = va[j]; b[j] = vb[j]; }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      a[j] = g + j < total ? lhs[g + j] : 0.f;
      b[j] = g + j < total ? rhs[g + j] : 0.f;
    }
  }
  const int64_t row_a = g / W;
  float w0, n0, w1 = 0.f, n1 = 0.f;
  merge_weights(lhs[row_a * W + W - 1], rhs[row_a * W + W - 1], w0, n0);
  const int64_t row_b = (g + 3) / W;
  if (row_b != row_a && row_b * W + W - 1 < total)
    merge_weights(lhs[row_b * W + W - 1], rhs[row_b * W + W - 1], w1, n1);
  float r[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t e = g + j;
    const bool second = e / W != row_a;
    const float w = second ? w1 : w0;
    const float nl = second ? n1 : n0;
    r[j] = (e % W == W - 1) ? nl : a[j] - w * (a[j] - b[j]);
  }
  if (g + 4 <= total) {
    f32x4 v = {r[0], r[1], r[2], r[3]};
    *reinterpret_cast<f32x4*>(dst + g) = v;
  } else {
    for (int j = 0; j < 4 && g + j < total; ++j) dst[g + j] = r[j];
  }
}

// Tree-attention merge of packed (rows x W) = (out | lse) operands across ranks
// (utils/flash_attn_dsl.py:307-324): with m = max over ranks of lse,
//   prepare: dst = (out * d | d),  d = exp(lse - m)      -- what every rank contributes to the SUM
//   finish:  dst = (sum_out / sum_d | m + log(sum_d))    -- from the summed contributions
// Packing d next to out * d makes the SUM one collective instead of the reference's two.  Rows whose
// lse is -inf everywhere (m = -inf) contribute d = 0 and finish as (0 | -inf).  Same flat walk in aligned
// groups of four floats as flash_reduce_kernel; `aux` is the per-row maximum, contiguous.
template <bool FINISH>
__global__ __launch_bounds__(256) void tree_merge_kernel(const float* __restrict__ src,
                                                         const float* __restrict__ aux,
                                                         float* __restrict__ dst, int64_t total, int W) {
  const int64_t g = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (g >= total) return;
  float a[4];
  if (g + 4 <= total) {
    const f32x4 va = *reinterpret_cast<const f32x4*>(src + g);
#pragma unroll
    for (int j = 0; j < 4; ++j) a[j] = va[j];
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) a[j] = g + j < total ? src[g + j] : 0.f;
  }
  const int64_t row_a = g / W;
  const int64_t row_b = (g + 3) / W;
  // per-row factor and last-column value, for the (at most) two rows this group touches
  float f[2] = {0.f, 0.f}, last[2] = {0.f, 0.f};
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const int64_t row = k == 0 ? row_a : row_b;
    if (k == 1 && (row_b == row_a || row_b * W + W - 1 >= total)) break;
    const float m = aux[row];
    const float tail = src[row * W + W - 1];
    if (!FINISH) {
      const float d = (m == -INFINITY) ? 0.f : __expf(tail - m);      // tail = this rank's lse
      f[k] = d;
      last[k] = d;
    } else {
      f[k] = tail > 0.f ? 1.f / tail : 0.f;                           // tail = summed d
      last[k] = tail > 0.f ? m + __logf(tail) : -INFINITY;
    }
  }
  float r[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t e = g + j;
    const int k = (e / W != row_a) ? 1 : 0;
    r[j] = (e % W == W - 1) ? last[k] : a[j] * f[k];
  }
  if (g + 4 <= total) {
    f32x4 v = {r[0], r[1], r[2], r[3]};
    *reinterpret_cast<f32x4*>(dst + g) = v;
  } else {
    for (int j = 0; j < 4 && g + j < total; ++j) dst[g + j] = r[j];
  }
}

// dst (rows x (D+1)) = pack(block)  or  flash_reduce(lhs, pack(block)); same flat walk over dst.
template <bool REDUCE>
__global__ __launch_bounds__(256) void pack_reduce_kernel(const float* __restrict__ lhs,
                                                          const uint16_t* __restrict__ block_out,
                                                          const float* __restrict__ block_lse,
                                                          float* __restrict__ dst,
                                                          int64_t total, int D, int Sq, int Hq) {
  const int W = D + 1;
  const int64_t g = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (g >= total) return;
  float r[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t e = g + j;
    if (e >= total) { r[j] = 0.f; continue; }
    const int64_t row = e / W;
    const int col = (int)(e % W);
    const int h = (int)(row % Hq);
    const int64_t bs = row / Hq;
    const int s = (int)(bs % Sq);
    const int64_t b = bs / Sq;
    const float bl = block_lse[(b * Hq + h) * Sq + s];
    float w = 1.f, nl = bl, a = 0.f;
    if (REDUCE) {
      merge_weights(lhs[row * W + D], bl, w, nl);
      a = lhs[e];
    }
    if (col == D) {
      r[j] = nl;
    } else {
      const float bo = bf16_lo(block_out[row * D + col]);
      r[j] = REDUCE ? a - w * (a - bo) : bo;
    }
  }
  if (g + 4 <= total) {
    f32x4 v = {r[0], r[1], r[2], r[3]};
    *reinterpret_cast<f32x4*>(dst + g) = v;
  } else {
    for (int j = 0; j < 4 && g + j < total; ++j) dst[g + j] = r[j];
  }
}

// ---- all blocks of a step at once --------------------------------------------------------------------
// The chunk loop of a ring step folds N block results into the accumulators one after the other
// (utils/flash_attn_dsl.py:51-71 called once per chunk, then the stores of :178-179), which moves the fp32
// accumulator through memory N - 1 times.  Folding is associative: with L = logsumexp_i(lse_i) the end
// result is out = sum_i exp(lse_i - L) * out_i, lse = L.  This kernel reads the N bf16 block outputs once
// and writes the bf16 output and the (B,H,S) LSE directly.  Rows whose lse is -inf everywhere give
// (0, -inf).  A block may cover only the rows s >= s_begin[i] of the sequence dimension (the zigzag
// schedule's "second half of the Q rows" steps); the rows before count as lse = -inf.
// One row = D/8 lanes x 8 contiguous head-dim values (16 bytes of bf16) per thread.
constexpr int kMaxBlocks = 16;
struct MergeManyParams {
  const uint16_t* out[kMaxBlocks];
  const float* lse[kMaxBlocks];
  uint16_t* final_out; float* final_lse;
  int s_begin[kMaxBlocks];        // first sequence row the block covers
  int64_t bo_sb[kMaxBlocks];      // batch stride of the block's output, elements
  int n, Sq, Hq;
  int64_t rows;
  int64_t bo_ss, bo_sh;
};

template <int LPR, int N>          // N = 0: run-time block count
__global__ __launch_bounds__(256) void lse_merge_many_kernel(const MergeManyParams p) {
  constexpr int D = LPR * 8;
  constexpr int kRowsPerPass = 256 / LPR;
  const int n = N > 0 ? N : p.n;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerPass + threadIdx.x / LPR;
  if (row >= p.rows) return;
  const int col = (threadIdx.x % LPR) * 8;
  const uint32_t h = (uint32_t)row % (uint32_t)p.Hq;
  const uint32_t bs = (uint32_t)row / (uint32_t)p.Hq;
  const uint32_t s = bs % (uint32_t)p.Sq;
  const uint32_t b = bs / (uint32_t)p.Sq;
  const int64_t l_off = ((int64_t)b * p.Hq + h) * p.Sq + s;
  u32x4 blk[N > 0 ? N : kMaxBlocks];
  float l[N > 0 ? N : kMaxBlocks];
#pragma unroll
  for (int i = 0; i < (N > 0 ? N : kMaxBlocks); ++i) {
    if (i < n) {
      const int sb = p.s_begin[i];
      l[i] = -INFINITY;
      blk[i] = u32x4{0u, 0u, 0u, 0u};
      if ((int)s >= sb) {
        const int64_t o_off = b * p.bo_sb[i] + (int64_t)(s - sb) * p.bo_ss + h * p.bo_sh + col;
        blk[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.out[i] + o_off));
        l[i] = p.lse[i][((int64_t)b * p.Hq + h) * (p.Sq - sb) + (s - sb)];
      }
    }
  }
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < (N > 0 ? N : kMaxBlocks); ++i)
    if (i < n) m = fmaxf(m, l[i]);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < (N > 0 ? N : kMaxBlocks); ++i) {
    if (i < n) {
      const float w = (m == -INFINITY) ? 0.f : __expf(l[i] - m);
      sum += w;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[2 * j] = __builtin_fmaf(w, bf16_lo(blk[i][j]), acc[2 * j]);
        acc[2 * j + 1] = __builtin_fmaf(w, bf16_hi(blk[i][j]), acc[2 * j + 1]);
      }
    }
  }
  const float inv = sum > 0.f ? 1.f / sum : 0.f;
  u32x4 w4;
#pragma unroll
  for (int j = 0; j < 4; ++j) w4[j] = pack_bf16(acc[2 * j] * inv, acc[2 * j + 1] * inv);
  *reinterpret_cast<u32x4*>(p.final_out + row * D + col) = w4;
  if (col == 0) p.final_lse[l_off] = sum > 0.f ? m + __logf(sum) : -INFINITY;
}

template <int LPR>
void launch_merge_many(const MergeManyParams& p, hipStream_t st) {
  constexpr int kRowsPerPass = 256 / LPR;
  const dim3 grid((unsigned)((p.rows + kRowsPerPass - 1) / kRowsPerPass)), block(256);
  if (p.n == 8) hipLaunchKernelGGL((lse_merge_many_kernel<LPR, 8>), grid, block, 0, st, p);
  else if (p.n == 4) hipLaunchKernelGGL((lse_merge_many_kernel<LPR, 4>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((lse_merge_many_kernel<LPR, 0>), grid, block, 0, st, p);
}

template <bool HAS_ACC>
__global__ __launch_bounds__(256) void grad_accumulate_kernel(const float* acc, const uint16_t* block,
                                                              float* dst, int64_t n) {
  const int64_t g = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (g >= n) return;
  if (g + 4 <= n) {
    const u32x2 w = *reinterpret_cast<const u32x2*>(block + g);
    f32x4 v = {bf16_lo(w[0]), bf16_hi(w[0]), bf16_lo(w[1]), bf16_hi(w[1])};
    if (HAS_ACC) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(acc + g);
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] += a[j];
    }
    *reinterpret_cast<f32x4*>(dst + g) = v;
  } else {
    for (int64_t e = g; e < n; ++e) dst[e] = (HAS_ACC ? acc[e] : 0.f) + bf16_lo(block[e]);
  }
}

}  // namespace

}  // namespace mhip

// ---- C ABI ----------------------------------------------------------------------------------------
using namespace mhip;

extern "C" int mhip_lse_merge(const float* acc_out, const float* acc_lse,
                              const void* block_out, const float* block_lse,
                              float* dst_out, float* dst_lse,
                              void* final_out, float* final_lse,
                              int B, int Sq, int Hq, int D,
                              int64_t ao_sb, int64_t ao_ss, int64_t ao_sh,
                              int64_t al_sb, int64_t al_ss, int64_t al_sh,
                              int64_t bo_sb, int64_t bo_ss, int64_t bo_sh,
                              int64_t bl_sb, int64_t bl_sh,
                              int64_t do_sb, int64_t do_ss, int64_t do_sh,
                              int64_t dl_sb, int64_t dl_ss, int64_t dl_sh,
                              void* stream) {
  if (B < 0 || Sq < 0 || Hq < 0 || D <= 0) return MHIP_EINVAL;
  if ((int64_t)B * Sq * Hq == 0) return MHIP_OK;
  if (!block_out || !block_lse) return MHIP_EINVAL;
  if ((acc_out == nullptr) != (acc_lse == nullptr)) return MHIP_EINVAL;
  if ((dst_out == nullptr) != (dst_lse == nullptr)) return MHIP_EINVAL;
  if ((final_out == nullptr) != (final_lse == nullptr)) return MHIP_EINVAL;
  if (!dst_out && !final_out) return MHIP_EINVAL;
  MergeParams p;
  p.acc_out = acc_out; p.acc_lse = acc_lse;
  p.block_out = static_cast<const uint16_t*>(block_out); p.block_lse = block_lse;
  p.dst_out = dst_out; p.dst_lse = dst_lse;
  p.final_out = static_cast<uint16_t*>(final_out); p.final_lse = final_lse;
  p.B = B; p.Sq = Sq; p.Hq = Hq; p.rows = (int64_t)B * Sq * Hq;
  p.ao_sb = ao_sb; p.ao_ss = ao_ss; p.ao_sh = ao_sh;
  p.al_sb = al_sb; p.al_ss = al_ss; p.al_sh = al_sh;
  p.bo_sb = bo_sb; p.bo_ss = bo_ss; p.bo_sh = bo_sh;
  p.bl_sb = bl_sb; p.bl_sh = bl_sh;
  p.do_sb = do_sb; p.do_ss = do_ss; p.do_sh = do_sh;
  p.dl_sb = dl_sb; p.dl_ss = dl_ss; p.dl_sh = dl_sh;
  const bool first = acc_out == nullptr, fin = final_out != nullptr;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // the vector kernel needs 16-byte aligned fp32 rows and 8-byte aligned bf16 rows
  auto mult4 = [](int64_t x) { return (x & 3) == 0; };
  bool vec = (D == 32 || D == 64 || D == 128 || D == 256) && p.rows < (int64_t(1) << 31) &&
             mult4(bo_sb) && mult4(bo_ss) && mult4(bo_sh) &&
             (reinterpret_cast<uintptr_t>(block_out) & 7u) == 0;
  if (!first) vec = vec && mult4(ao_sb) && mult4(ao_ss) && mult4(ao_sh) && aligned16(acc_out);
  if (dst_out) vec = vec && mult4(do_sb) && mult4(do_ss) && mult4(do_sh) && aligned16(dst_out);
  if (fin) vec = vec && (reinterpret_cast<uintptr_t>(final_out) & 7u) == 0;
  auto mult8 = [](int64_t x) { return (x & 7) == 0; };
  const bool vec8 = vec && !first && D == 128 && mult8(bo_sb) && mult8(bo_ss) && mult8(bo_sh) && aligned16(block_out) &&
                    (!fin || aligned16(final_out));
  if (vec8) {
    launch_merge8<16>(p, first, fin, st);
  } else if (vec) {
    switch (D) {
      case 32: launch_merge<8>(p, first, fin, st); break;
      case 64: launch_merge<16>(p, first, fin, st); break;
      case 128: launch_merge<32>(p, first, fin, st); break;
      default: launch_merge<64>(p, first, fin, st); break;
    }
  } else {
    const int64_t n = p.rows * D;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (first && fin) hipLaunchKernelGGL((lse_merge_generic<true, true>), grid, block, 0, st, p, D);
    else if (first) hipLaunchKernelGGL((lse_merge_generic<true, false>), grid, block, 0, st, p, D);
    else if (fin) hipLaunchKernelGGL((lse_merge_generic<false, true>), grid, block, 0, st, p, D);
    else hipLaunchKernelGGL((lse_merge_generic<false, false>), grid, block, 0, st, p, D);
  }
  return launch_status();
}

extern "C" int mhip_lse_merge_many(const void* const* block_outs, const float* const* block_lses,
                                   const int64_t* bo_sb, const int* s_begin, int n,
                                   void* final_out, float* final_lse,
                                   int B, int Sq, int Hq, int D,
                                   int64_t bo_ss, int64_t bo_sh, void* stream) {
  if (B < 0 || Sq < 0 || Hq < 0 || D <= 0 || n < 1 || n > kMaxBlocks) return MHIP_EINVAL;
  if (D != 64 && D != 128 && D != 256) return MHIP_EUNSUPPORTED;
  const int64_t rows = (int64_t)B * Sq * Hq;
  if (rows == 0) return MHIP_OK;
  if (rows >= (int64_t(1) << 31)) return MHIP_EUNSUPPORTED;
  if (!block_outs || !block_lses || !bo_sb || !final_out || !final_lse) return MHIP_EINVAL;
  if ((bo_ss & 7) || (bo_sh & 7)) return MHIP_EALIGN;
  if (!aligned16(final_out)) return MHIP_EALIGN;
  MergeManyParams p;
  for (int i = 0; i < kMaxBlocks; ++i) { p.out[i] = nullptr; p.lse[i] = nullptr; p.s_begin[i] = 0; p.bo_sb[i] = 0; }
  for (int i = 0; i < n; ++i) {
    if (!block_outs[i] || !block_lses[i]) return MHIP_EINVAL;
    const int sb = s_begin ? s_begin[i] : 0;
    if (sb < 0 || sb > Sq) return MHIP_EINVAL;
    if (!aligned16(block_outs[i]) || (bo_sb[i] & 7)) return MHIP_EALIGN;
    p.s_begin[i] = sb;
    p.bo_sb[i] = bo_sb[i];
    p.out[i] = static_cast<const uint16_t*>(block_outs[i]);
    p.lse[i] = block_lses[i];
  }
  p.final_out = static_cast<uint16_t*>(final_out); p.final_lse = final_lse;
  p.n = n; p.Sq = Sq; p.Hq = Hq; p.rows = rows;
  p.bo_ss = bo_ss; p.bo_sh = bo_sh;
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (D) {
    case 64: launch_merge_many<8>(p, st); break;
    case 128: launch_merge_many<16>(p, st); break;
    default: launch_merge_many<32>(p, st); break;
  }
  return launch_status();
}

extern "C" int mhip_flash_reduce(const float* lhs, const float* rhs, float* dst,
                                 int64_t rows, int D, void* stream) {
  if (rows < 0 || D <= 0) return MHIP_EINVAL;
  if (rows == 0) return MHIP_OK;
  if (!lhs || !rhs || !dst) return MHIP_EINVAL;
  if (!aligned16(lhs) || !aligned16(rhs) || !aligned16(dst)) return MHIP_EALIGN;
  const int64_t total = rows * (D + 1);
  const int64_t groups = (total + 3) / 4;
  hipLaunchKernelGGL(flash_reduce_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), lhs, rhs, dst, total, D + 1);
  return launch_status();
}

extern "C" int mhip_tree_merge(const float* src, const float* row_max, float* dst, int64_t rows, int D,
                               int finish, void* stream) {
  if (rows < 0 || D <= 0) return MHIP_EINVAL;
  if (rows == 0) return MHIP_OK;
  if (!src || !row_max || !dst) return MHIP_EINVAL;
  if (!aligned16(src) || !aligned16(dst)) return MHIP_EALIGN;
  const int64_t total = rows * (D + 1);
  const int64_t groups = (total + 3) / 4;
  const dim3 grid((unsigned)((groups + 255) / 256)), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (finish) hipLaunchKernelGGL(tree_merge_kernel<true>, grid, block, 0, st, src, row_max, dst, total, D + 1);
  else hipLaunchKernelGGL(tree_merge_kernel<false>, grid, block, 0, st, src, row_max, dst, total, D + 1);
  return launch_status();
}

extern "C" int mhip_pack_reduce(const float* lhs, const void* block_out, const float* block_lse,
                                float* dst, int B, int Sq, int Hq, int D, void* stream) {
  if (B < 0 || Sq < 0 || Hq < 0 || D <= 0) return MHIP_EINVAL;
  const int64_t rows = (int64_t)B * Sq * Hq;
  if (rows == 0) return MHIP_OK;
  if (!block_out || !block_lse || !dst) return MHIP_EINVAL;
  if (!aligned16(dst)) return MHIP_EALIGN;
  const int64_t total = rows * (D + 1);
  const int64_t groups = (total + 3) / 4;
  const dim3 grid((unsigned)((groups + 255) / 256)), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (lhs)
    hipLaunchKernelGGL(pack_reduce_kernel<true>, grid, block, 0, st, lhs,
                       static_cast<const uint16_t*>(block_out), block_lse, dst, total, D, Sq, Hq);
  else
    hipLaunchKernelGGL(pack_reduce_kernel<false>, grid, block, 0, st, lhs,
                       static_cast<const uint16_t*>(block_out), block_lse, dst, total, D, Sq, Hq);
  return launch_status();
}

extern "C" int mhip_grad_accumulate(const float* acc, const void* block, float* dst, int64_t n,
                                    void* stream) {
  if (n < 0) return MHIP_EINVAL;
  if (n == 0) return MHIP_OK;
  if (!block || !dst) return MHIP_EINVAL;
  if (!aligned16(dst) || (acc && !aligned16(acc)) || (reinterpret_cast<uintptr_t>(block) & 7u))
    return MHIP_EALIGN;
  const int64_t groups = (n + 3) / 4;
  const dim3 grid((unsigned)((groups + 255) / 256)), block_dim(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (acc)
    hipLaunchKernelGGL(grad_accumulate_kernel<true>, grid, block_dim, 0, st, acc,
                       static_cast<const uint16_t*>(block), dst, n);
  else
    hipLaunchKernelGGL(grad_accumulate_kernel<false>, grid, block_dim, 0, st, acc,
                       static_cast<const uint16_t*>(block), dst, n);
  return launch_status();
}
