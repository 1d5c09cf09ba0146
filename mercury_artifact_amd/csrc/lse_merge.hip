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

// Accumulator traffic: plain loads, non-temporal stores (non-temporal loads measured slower, plain stores too).
__device__ __forceinline__ f32x4 stream_load(const f32x4* p) { return *p; }
__device__ __forceinline__ void stream_store(f32x4 v, f32x4* p) { __builtin_nontemporal_store(v, p); }

struct MergeParams {
  const float* acc_out; const float* acc_lse;
  const uint16_t* block_out; const float* block_lse;
  float* dst_out; float* dst_lse;
  uint16_t* final_out; float* final_lse;
  int B, Sq, Hq;
  int D;             // head dimension (the vector kernels: a multiple of 4; a row takes LPR >= D / 4 lanes)
  int64_t rows;
  int64_t ao_sb, ao_ss, ao_sh, al_sb, al_ss, al_sh, bo_sb, bo_ss, bo_sh, bl_sb, bl_sh;
  int64_t do_sb, do_ss, do_sh, dl_sb, dl_ss, dl_sh;
};

// One row = LPR lanes x 4 contiguous head-dim values (lanes past the head dimension idle: LPR is the power of two
// that holds D / 4), ROWS rows per thread.  Measured on MI355X at
// 131072 rows x 128: two rows per thread with non-temporal stores is the fastest setting (5.8 TB/s in
// place, 5.2 TB/s into a separate destination); more rows per thread or non-temporal loads are slower.
template <int LPR, int ROWS, bool FIRST, bool FINAL>
__global__ __launch_bounds__(256) void lse_merge_kernel(const MergeParams p) {
  const int D = p.D;
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
    live[r] = row < p.rows && col < D;
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

// Generic head dimension or unaligned operands: one row per 32 lanes of one wavefront, the lanes stepping
// through the columns.  dst may alias acc: an output element is read and written by the same lane only, and
// the row's lse is loaded by all lanes of the row in one instruction before the one lane that owns it stores
// the new value, which depends on that load (so the load has returned for the whole wavefront).
constexpr int kGenericLanes = 32;
template <bool FIRST, bool FINAL>
__global__ __launch_bounds__(256) void lse_merge_generic(const MergeParams p, int D) {
  const int64_t row = (int64_t)blockIdx.x * (256 / kGenericLanes) + threadIdx.x / kGenericLanes;
  if (row >= p.rows) return;
  const int lane = threadIdx.x % kGenericLanes;
  const int h = (int)(row % p.Hq);
  const int64_t bs = row / p.Hq;
  const int s = (int)(bs % p.Sq);
  const int b = (int)(bs / p.Sq);
  const float bl = p.block_lse[b * p.bl_sb + h * p.bl_sh + s];
  float w = 1.f, new_lse = bl;
  if (!FIRST) merge_weights(p.acc_lse[b * p.al_sb + s * p.al_ss + h * p.al_sh], bl, w, new_lse);
  const uint16_t* bo_row = p.block_out + b * p.bo_sb + s * p.bo_ss + h * p.bo_sh;
  const float* a_row = FIRST ? nullptr : p.acc_out + b * p.ao_sb + s * p.ao_ss + h * p.ao_sh;
  float* d_row = p.dst_out ? p.dst_out + b * p.do_sb + s * p.do_ss + h * p.do_sh : nullptr;
  for (int col = lane; col < D; col += kGenericLanes) {
    const float bo = bf16_lo(bo_row[col]);
    float res = bo;
    if (!FIRST) {
      const float a = a_row[col];
      res = a - w * (a - bo);
    }
    if (d_row) d_row[col] = res;
    if (FINAL) p.final_out[row * D + col] = (uint16_t)(pack_bf16(res, 0.f) & 0xffffu);
  }
  if (lane == 0) {
    if (d_row) p.dst_lse[b * p.dl_sb + s * p.dl_ss + h * p.dl_sh] = new_lse;
    if (FINAL) p.final_lse[((int64_t)b * p.Hq + h) * p.Sq + s] = new_lse;
  }
}

template <int LPR>
void launch_merge(const MergeParams& p, bool first, bool fin, hipStream_t st) {
  constexpr int ROWS = 2;            // rows in flight per thread (1 and 4 measured slower)
  constexpr int kRowsPerBlock = (256 / LPR) * ROWS;
  const dim3 grid((unsigned)((p.rows + kRowsPerBlock - 1) / kRowsPerBlock)), block(256);
  if (first && fin) hipLaunchKernelGGL((lse_merge_kernel<LPR, ROWS, true, true>), grid, block, 0, st, p);
  else if (first) hipLaunchKernelGGL((lse_merge_kernel<LPR, ROWS, true, false>), grid, block, 0, st, p);
  else if (fin) hipLaunchKernelGGL((lse_merge_kernel<LPR, ROWS, false, true>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((lse_merge_kernel<LPR, ROWS, false, false>), grid, block, 0, st, p);
}

// The same merge with eight head-dim values per lane: one 16-byte load of the bf16 block row piece, two
// 16-byte loads and stores of the fp32 accumulator.  Measured at 131072 rows x 128 against the kernel
// above, launches back to back: 29.1 vs 30.5 us into a separate destination, 28.0 vs 29.2 us in place,
// 21.9 vs 29.8 us with the fused bf16 epilogue, 21.1 vs 16.8 us for the first-call cast.  Inside a ring
// step, where a merge follows a block forward and its operands were written just before, the plain merge
// is faster with four values per lane (31.6 vs 33.4 us), so only the fused-epilogue merges run here.
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
    live[r] = row < p.rows && col < D;
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
  constexpr int ROWS = 1;
  constexpr int kRowsPerBlock = (256 / LPR) * ROWS;
  const dim3 grid((unsigned)((p.rows + kRowsPerBlock - 1) / kRowsPerBlock)), block(256);
  if (first && fin) hipLaunchKernelGGL((lse_merge_kernel8<LPR, ROWS, true, true>), grid, block, 0, st, p);
  else if (first) hipLaunchKernelGGL((lse_merge_kernel8<LPR, ROWS, true, false>), grid, block, 0, st, p);
  else if (fin) hipLaunchKernelGGL((lse_merge_kernel8<LPR, ROWS, false, true>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((lse_merge_kernel8<LPR, ROWS, false, false>), grid, block, 0, st, p);
}

// ---- packed form -----------------------------------------------------------------------------------
// flash_reduce (utils/flash_attn_dsl.py:293-305), the pack that feeds it (utils/flash_attn_dsl.py:396) and
// the tree-attention merge (utils/flash_attn_dsl.py:307-324) work on flat fp32 arrays of rows x (D+1),
// the LSE in the last column.  A row is 4(D+1) bytes long, which is not a multiple of 16 for D = 128, so
// the kernels walk the flat array in aligned groups of four floats: one division per thread (by a
// compile-time row width when D = 128) places the group, and its four elements sit in at most two rows,
// found by stepping.  Threads read the LSE column of rows whose other elements belong to other threads,
// so dst must not overlap the inputs.  IT is the index type: 32 bits for buffers of fewer than 2^31
// elements, 64 bits otherwise.
//
// Tree-attention merge: with m = max over ranks of lse,
//   prepare: dst = (out * d | d),  d = exp(lse - m)      -- what every rank contributes to the SUM
//   finish:  dst = (sum_out / sum_d | m + log(sum_d))    -- from the summed contributions
// Packing d next to out * d makes the SUM one collective instead of the reference's two.  Rows whose
// lse is -inf everywhere (m = -inf) contribute d = 0 and finish as (0 | -inf).  `aux` is the per-row
// maximum, contiguous.
template <typename IT>
struct PackedPos {
  IT row;                 // of the group's first element
  uint32_t col;
};
template <int WCT, typename IT>
__device__ __forceinline__ PackedPos<IT> packed_pos(IT g, uint32_t w_rt) {
  const uint32_t W = WCT ? (uint32_t)WCT : w_rt;
  PackedPos<IT> p;
  p.row = g / W;
  p.col = (uint32_t)(g - p.row * W);
  return p;
}
template <typename IT>
__device__ __forceinline__ f32x4 load4(const float* base, IT g, IT total) {
  if (g + 4 <= total) return *reinterpret_cast<const f32x4*>(base + g);
  f32x4 v = {0.f, 0.f, 0.f, 0.f};
  for (IT j = 0; j < 4 && g + j < total; ++j) v[j] = base[g + j];
  return v;
}
template <typename IT>
__device__ __forceinline__ void store4(float* base, IT g, IT total, const f32x4& v) {
  if (g + 4 <= total) { *reinterpret_cast<f32x4*>(base + g) = v; return; }
  for (IT j = 0; j < 4 && g + j < total; ++j) base[g + j] = v[j];
}

template <int WCT, typename IT>
__global__ __launch_bounds__(256) void flash_reduce_kernel(const float* __restrict__ lhs, const float* __restrict__ rhs,
                                                           float* __restrict__ dst, IT total, uint32_t w_rt) {
  const uint32_t W = WCT ? (uint32_t)WCT : w_rt;
  const IT g = ((IT)blockIdx.x * 256u + threadIdx.x) * 4u;
  if (g >= total) return;
  const PackedPos<IT> pos = packed_pos<WCT, IT>(g, w_rt);
  const f32x4 a = load4<IT>(lhs, g, total), b = load4<IT>(rhs, g, total);
  float w[2] = {0.f, 0.f}, nl[2] = {0.f, 0.f};
  const IT last0 = pos.row * W + W - 1;
  merge_weights(lhs[last0], rhs[last0], w[0], nl[0]);
  if (pos.col + 3 >= W && last0 + W < total) merge_weights(lhs[last0 + W], rhs[last0 + W], w[1], nl[1]);
  f32x4 r;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t c = pos.col + j;
    const int k = c >= W ? 1 : 0;
    const uint32_t cc = k ? c - W : c;
    r[j] = cc == W - 1 ? nl[k] : a[j] - w[k] * (a[j] - b[j]);
  }
  store4<IT>(dst, g, total, r);
}

template <bool FINISH, int WCT, typename IT>
__global__ __launch_bounds__(256) void tree_merge_kernel(const float* __restrict__ src, const float* __restrict__ aux,
                                                         float* __restrict__ dst, IT total, uint32_t w_rt) {
  const uint32_t W = WCT ? (uint32_t)WCT : w_rt;
  const IT g = ((IT)blockIdx.x * 256u + threadIdx.x) * 4u;
  if (g >= total) return;
  const PackedPos<IT> pos = packed_pos<WCT, IT>(g, w_rt);
  const f32x4 a = load4<IT>(src, g, total);
  float f[2] = {0.f, 0.f}, last[2] = {0.f, 0.f};
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const IT row = pos.row + k;
    if (k == 1 && !(pos.col + 3 >= W && row * W + W - 1 < total)) break;
    const float m = aux[row];
    const float tail = src[row * W + W - 1];
    if (!FINISH) {
      const float d = (m == -INFINITY) ? 0.f : __expf(tail - m);
      f[k] = d;
      last[k] = d;
    } else {
      f[k] = tail > 0.f ? 1.f / tail : 0.f;
      last[k] = tail > 0.f ? m + __logf(tail) : -INFINITY;
    }
  }
  f32x4 r;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t c = pos.col + j;
    const int k = c >= W ? 1 : 0;
    const uint32_t cc = k ? c - W : c;
    r[j] = cc == W - 1 ? last[k] : a[j] * f[k];
  }
  store4<IT>(dst, g, total, r);
}

// The same for dst == src (the natural use: all-reduce the packed buffer in place, finish in place).  The
// flat walk above reads a row's last column from a thread that does not own it, so in place it would race
// with the owner's store; here one row belongs to 32 lanes of one wavefront, which all load the last column
// in one instruction before the lane that owns it stores the new value computed from that load.
template <bool FINISH>
__global__ __launch_bounds__(256) void tree_merge_rows_kernel(const float* src, const float* __restrict__ aux,
                                                              float* dst, int64_t rows, uint32_t W) {
  const int64_t row = (int64_t)blockIdx.x * (256 / kGenericLanes) + threadIdx.x / kGenericLanes;
  if (row >= rows) return;
  const uint32_t lane = threadIdx.x % kGenericLanes;
  const float m = aux[row];
  const float tail = src[row * W + W - 1];
  float f, last;
  if (!FINISH) {
    f = (m == -INFINITY) ? 0.f : __expf(tail - m);
    last = f;
  } else {
    f = tail > 0.f ? 1.f / tail : 0.f;
    last = tail > 0.f ? m + __logf(tail) : -INFINITY;
  }
  for (uint32_t c = lane; c + 1 < W; c += kGenericLanes) dst[row * W + c] = src[row * W + c] * f;
  if (lane == 0) dst[row * W + W - 1] = last;
}

template <bool REDUCE, int WCT, typename IT>
__global__ __launch_bounds__(256) void pack_reduce_kernel(const float* __restrict__ lhs,
                                                          const uint16_t* __restrict__ block_out,
                                                          const float* __restrict__ block_lse,
                                                          float* __restrict__ dst, IT total, uint32_t w_rt,
                                                          uint32_t Sq, uint32_t Hq) {
  const uint32_t W = WCT ? (uint32_t)WCT : w_rt, D = W - 1;
  const IT g = ((IT)blockIdx.x * 256u + threadIdx.x) * 4u;
  if (g >= total) return;
  const PackedPos<IT> pos = packed_pos<WCT, IT>(g, w_rt);
  uint32_t h = (uint32_t)(pos.row % Hq);
  const IT bs = pos.row / Hq;
  uint32_t s = (uint32_t)(bs % Sq);
  IT b = bs / Sq;
  f32x4 a = {0.f, 0.f, 0.f, 0.f};
  if (REDUCE) a = load4<IT>(lhs, g, total);
  float w[2] = {1.f, 1.f}, nl[2] = {0.f, 0.f};
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const IT row = pos.row + k;
    if (k == 1) {
      if (!(pos.col + 3 >= W && row * W < total)) break;
      if (++h == Hq) { h = 0; if (++s == Sq) { s = 0; ++b; } }
    }
    const float bl = block_lse[(b * Hq + h) * Sq + s];
    nl[k] = bl;
    if (REDUCE) merge_weights(lhs[row * W + D], bl, w[k], nl[k]);
  }
  f32x4 r;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t c = pos.col + j;
    const int k = c >= W ? 1 : 0;
    const uint32_t cc = k ? c - W : c;
    if (g + j >= total) { r[j] = 0.f; continue; }
    if (cc == D) {
      r[j] = nl[k];
    } else {
      const float bo = bf16_lo(block_out[(pos.row + k) * D + cc]);
      r[j] = REDUCE ? a[j] - w[k] * (a[j] - bo) : bo;
    }
  }
  store4<IT>(dst, g, total, r);
}

// Epilogue of the packed form (utils/flash_attn_dsl.py:406-407 after the managed reduction: the output is
// buf[..., :-1] cast to the query's type, the LSE buf[..., -1] transposed to (B,H,S)): one row per D/8 lanes,
// eight 4-byte loads (a packed row starts on a 4-byte boundary only) and one 16-byte store per lane.
__global__ __launch_bounds__(256) void unpack_kernel(const float* __restrict__ buf, uint16_t* __restrict__ out,
                                                     float* __restrict__ lse, uint32_t rows, uint32_t D,
                                                     uint32_t Sq, uint32_t Hq) {
  const uint32_t lpr = D / 8;
  const uint32_t row = (blockIdx.x * 256u + threadIdx.x) / lpr;
  if (row >= rows) return;
  const uint32_t col = ((blockIdx.x * 256u + threadIdx.x) % lpr) * 8;
  const float* src = buf + (uint64_t)row * (D + 1) + col;
  u32x4 w;
#pragma unroll
  for (int j = 0; j < 4; ++j) w[j] = pack_bf16(src[2 * j], src[2 * j + 1]);
  *reinterpret_cast<u32x4*>(out + (uint64_t)row * D + col) = w;
  if (col == 0) {
    const uint32_t h = row % Hq, bs = row / Hq, s = bs % Sq, b = bs / Sq;
    lse[((uint64_t)b * Hq + h) * Sq + s] = buf[(uint64_t)row * (D + 1) + D];
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
// More than kGroup blocks are folded in groups of kGroup with the running (maximum, sum, weighted output) carried
// in registers, the online-softmax way, still in one pass over every block.
constexpr int kMaxBlocks = 64;
constexpr int kGroup = 16;
struct MergeManyParams {
  const uint16_t* out[kMaxBlocks];
  const float* lse[kMaxBlocks];
  uint16_t* final_out; float* final_lse;
  int s_begin[kMaxBlocks];        // first sequence row the block covers
  int64_t bo_sb[kMaxBlocks];      // batch stride of the block's output, elements
  int n, Sq, Hq;
  int D;                          // head dimension, a multiple of 8; a row takes LPR >= D / 8 lanes (a power of two)
  int64_t rows;
  int64_t bo_ss, bo_sh;
};

template <int LPR, int N>          // N = 0: run-time block count, folded in groups of kGroup
__global__ __launch_bounds__(256) void lse_merge_many_kernel(const MergeManyParams p) {
  const int D = p.D;
  constexpr int kRowsPerPass = 256 / LPR;
  constexpr int G = N > 0 ? N : kGroup;
  const int n = N > 0 ? N : p.n;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerPass + threadIdx.x / LPR;
  if (row >= p.rows) return;
  const int col = (threadIdx.x % LPR) * 8;
  if (col >= D) return;            // head dimensions that do not fill the row's lanes (no cross-lane work below)
  const uint32_t h = (uint32_t)row % (uint32_t)p.Hq;
  const uint32_t bs = (uint32_t)row / (uint32_t)p.Hq;
  const uint32_t s = bs % (uint32_t)p.Sq;
  const uint32_t b = bs / (uint32_t)p.Sq;
  const int64_t l_off = ((int64_t)b * p.Hq + h) * p.Sq + s;
  float m = -INFINITY;             // maximum of the lse folded so far
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float sum = 0.f;                 // both relative to m
  for (int g0 = 0; g0 < n; g0 += G) {
    u32x4 blk[G];
    float l[G];
#pragma unroll
    for (int i = 0; i < G; ++i) {
      l[i] = -INFINITY;
      blk[i] = u32x4{0u, 0u, 0u, 0u};
      if (g0 + i < n) {
        const int sb = p.s_begin[g0 + i];
        if ((int)s >= sb) {
          const int64_t o_off = b * p.bo_sb[g0 + i] + (int64_t)(s - sb) * p.bo_ss + h * p.bo_sh + col;
          blk[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.out[g0 + i] + o_off));
          l[i] = p.lse[g0 + i][((int64_t)b * p.Hq + h) * (p.Sq - sb) + (s - sb)];
        }
      }
    }
    float m_new = m;
#pragma unroll
    for (int i = 0; i < G; ++i) m_new = fmaxf(m_new, l[i]);
    if (N == 0 && g0 > 0) {
      // what was folded before this group moves to the new maximum (exp(-inf - x) = 0 handles an empty past)
      const float carry = (m_new == -INFINITY) ? 0.f : __expf(m - m_new);
      sum *= carry;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] *= carry;
    }
    m = m_new;
#pragma unroll
    for (int i = 0; i < G; ++i) {
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
  p.D = D;
  bool vec = (D & 3) == 0 && D <= 256 && p.rows < (int64_t(1) << 31) &&
             mult4(bo_sb) && mult4(bo_ss) && mult4(bo_sh) &&
             (reinterpret_cast<uintptr_t>(block_out) & 7u) == 0;
  if (!first) vec = vec && mult4(ao_sb) && mult4(ao_ss) && mult4(ao_sh) && aligned16(acc_out);
  if (dst_out) vec = vec && mult4(do_sb) && mult4(do_ss) && mult4(do_sh) && aligned16(dst_out);
  if (fin) vec = vec && (reinterpret_cast<uintptr_t>(final_out) & 7u) == 0;
  auto mult8 = [](int64_t x) { return (x & 7) == 0; };
  // eight values per lane pay for the merges with the fused bf16 epilogue only (the others measured slower in the chain)
  const bool vec8 = fin && vec && !first && D == 128 && mult8(bo_sb) && mult8(bo_ss) && mult8(bo_sh) && aligned16(block_out) &&
                    (!fin || aligned16(final_out));
  if (vec8) {
    launch_merge8<16>(p, first, fin, st);
  } else if (vec) {
    // lanes per row: the power of two that holds D / 4 (all lanes busy at D = 32, 64, 128, 256)
    if (D <= 32) launch_merge<8>(p, first, fin, st);
    else if (D <= 64) launch_merge<16>(p, first, fin, st);
    else if (D <= 128) launch_merge<32>(p, first, fin, st);
    else launch_merge<64>(p, first, fin, st);
  } else {
    constexpr int kRowsPerBlock = 256 / kGenericLanes;
    if (p.rows / kRowsPerBlock >= (int64_t(1) << 31)) return MHIP_EUNSUPPORTED;
    const dim3 grid((unsigned)((p.rows + kRowsPerBlock - 1) / kRowsPerBlock)), block(256);
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
  if (D > 256 || (D & 7) != 0) return MHIP_EUNSUPPORTED;
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
  p.n = n; p.Sq = Sq; p.Hq = Hq; p.D = D; p.rows = rows;
  p.bo_ss = bo_ss; p.bo_sh = bo_sh;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // lanes per row: the power of two that holds D / 8 (all lanes busy at D = 32, 64, 128, 256)
  if (D <= 32) launch_merge_many<4>(p, st);
  else if (D <= 64) launch_merge_many<8>(p, st);
  else if (D <= 128) launch_merge_many<16>(p, st);
  else launch_merge_many<32>(p, st);
  return launch_status();
}

extern "C" int mhip_flash_reduce(const float* lhs, const float* rhs, float* dst,
                                 int64_t rows, int D, void* stream) {
  if (rows < 0 || D <= 0) return MHIP_EINVAL;
  if (rows == 0) return MHIP_OK;
  if (!lhs || !rhs || !dst) return MHIP_EINVAL;
  if (!aligned16(lhs) || !aligned16(rhs) || !aligned16(dst)) return MHIP_EALIGN;
  const int64_t total = rows * (D + 1);
  if ((dst < lhs + total && lhs < dst + total) || (dst < rhs + total && rhs < dst + total)) return MHIP_EINVAL;
  const int64_t groups = (total + 3) / 4;
  const dim3 grid((unsigned)((groups + 255) / 256)), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint32_t w = (uint32_t)(D + 1);
  if (total < (int64_t(1) << 31)) {
    if (D == 128) hipLaunchKernelGGL((flash_reduce_kernel<129, uint32_t>), grid, block, 0, st, lhs, rhs, dst, (uint32_t)total, w);
    else hipLaunchKernelGGL((flash_reduce_kernel<0, uint32_t>), grid, block, 0, st, lhs, rhs, dst, (uint32_t)total, w);
  } else {
    hipLaunchKernelGGL((flash_reduce_kernel<0, uint64_t>), grid, block, 0, st, lhs, rhs, dst, (uint64_t)total, w);
  }
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
  const uint32_t w = (uint32_t)(D + 1);
  if (dst == src) {
    constexpr int kRowsPerBlock = 256 / kGenericLanes;
    if (rows / kRowsPerBlock >= (int64_t(1) << 31)) return MHIP_EUNSUPPORTED;
    const dim3 rgrid((unsigned)((rows + kRowsPerBlock - 1) / kRowsPerBlock));
    if (finish) hipLaunchKernelGGL(tree_merge_rows_kernel<true>, rgrid, block, 0, st, src, row_max, dst, rows, w);
    else hipLaunchKernelGGL(tree_merge_rows_kernel<false>, rgrid, block, 0, st, src, row_max, dst, rows, w);
    return launch_status();
  }
  if (dst < src + total && src < dst + total) return MHIP_EINVAL;      // partial overlap
  if (total < (int64_t(1) << 31)) {
    const uint32_t t32 = (uint32_t)total;
    if (finish && D == 128) hipLaunchKernelGGL((tree_merge_kernel<true, 129, uint32_t>), grid, block, 0, st, src, row_max, dst, t32, w);
    else if (finish) hipLaunchKernelGGL((tree_merge_kernel<true, 0, uint32_t>), grid, block, 0, st, src, row_max, dst, t32, w);
    else if (D == 128) hipLaunchKernelGGL((tree_merge_kernel<false, 129, uint32_t>), grid, block, 0, st, src, row_max, dst, t32, w);
    else hipLaunchKernelGGL((tree_merge_kernel<false, 0, uint32_t>), grid, block, 0, st, src, row_max, dst, t32, w);
  } else if (finish) {
    hipLaunchKernelGGL((tree_merge_kernel<true, 0, uint64_t>), grid, block, 0, st, src, row_max, dst, (uint64_t)total, w);
  } else {
    hipLaunchKernelGGL((tree_merge_kernel<false, 0, uint64_t>), grid, block, 0, st, src, row_max, dst, (uint64_t)total, w);
  }
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
  const uint16_t* bo = static_cast<const uint16_t*>(block_out);
  if (lhs && !aligned16(lhs)) return MHIP_EALIGN;
  if (lhs && dst < lhs + total && lhs < dst + total) return MHIP_EINVAL;
  const uint32_t w = (uint32_t)(D + 1), sq = (uint32_t)Sq, hq = (uint32_t)Hq;
  if (total < (int64_t(1) << 31)) {
    const uint32_t t32 = (uint32_t)total;
    if (lhs && D == 128) hipLaunchKernelGGL((pack_reduce_kernel<true, 129, uint32_t>), grid, block, 0, st, lhs, bo, block_lse, dst, t32, w, sq, hq);
    else if (lhs) hipLaunchKernelGGL((pack_reduce_kernel<true, 0, uint32_t>), grid, block, 0, st, lhs, bo, block_lse, dst, t32, w, sq, hq);
    else if (D == 128) hipLaunchKernelGGL((pack_reduce_kernel<false, 129, uint32_t>), grid, block, 0, st, lhs, bo, block_lse, dst, t32, w, sq, hq);
    else hipLaunchKernelGGL((pack_reduce_kernel<false, 0, uint32_t>), grid, block, 0, st, lhs, bo, block_lse, dst, t32, w, sq, hq);
  } else if (lhs) {
    hipLaunchKernelGGL((pack_reduce_kernel<true, 0, uint64_t>), grid, block, 0, st, lhs, bo, block_lse, dst, (uint64_t)total, w, sq, hq);
  } else {
    hipLaunchKernelGGL((pack_reduce_kernel<false, 0, uint64_t>), grid, block, 0, st, lhs, bo, block_lse, dst, (uint64_t)total, w, sq, hq);
  }
  return launch_status();
}

extern "C" int mhip_unpack(const float* buf, void* out, float* lse, int B, int Sq, int Hq, int D, void* stream) {
  if (B < 0 || Sq < 0 || Hq < 0 || D <= 0) return MHIP_EINVAL;
  if (D % 8 != 0 || 256 % (D / 8) != 0) return MHIP_EUNSUPPORTED;
  const int64_t rows = (int64_t)B * Sq * Hq;
  if (rows == 0) return MHIP_OK;
  if (rows >= (int64_t(1) << 31) / (D / 8)) return MHIP_EUNSUPPORTED;
  if (!buf || !out || !lse) return MHIP_EINVAL;
  if (!aligned16(out) || (reinterpret_cast<uintptr_t>(buf) & 3u)) return MHIP_EALIGN;
  const int64_t threads = rows * (D / 8);
  hipLaunchKernelGGL(unpack_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), buf, static_cast<uint16_t*>(out), lse, (uint32_t)rows,
                     (uint32_t)D, (uint32_t)Sq, (uint32_t)Hq);
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
