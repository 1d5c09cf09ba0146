// Block backward of the ring-attention step for gfx950, recomputing P from the saved LSE.
//
// Replaces the flash-attn call at utils/attn_bwd_dsl.py:83-115 of the reference:
//     P = exp(scale * q k^T - lse),  delta = rowsum(dout * out)
//     dV = P^T dout,  dP = dout v^T,  dS = P * (dP - delta),  dQ = scale * dS k,  dK = scale * dS^T q
//
// Three kernels, no atomics (so every run is deterministic):
//   bwd_delta    delta[b,h,i] = sum_d dout * out                        (bandwidth bound)
//   bwd_main<DQ=false>  one workgroup per 128 keys of one KV head: K and V rows stay in registers,
//                Q / dout tiles of the (grouped) query heads stream through LDS; accumulates dK, dV
//   bwd_main<DQ=true>   one workgroup per 128 query rows of one head: Q and dout rows stay in registers,
//                K / V tiles stream through LDS; accumulates dQ
// Both instances share one body.  "Stationary" rows (32 per wavefront) sit in the lane index of every
// MFMA accumulator, "streamed" rows in its registers, exactly as in the forward kernel:
//     T1[c][r] = X_str[c] . X_st[r]      (scores)          T2[c][r] = Y_str[c] . Y_st[r]      (dP)
//     acc^T[d][r] += X_str^T[d][c] dS[c][r]                (dQ or dK)
//     acc2^T[d][r] += Y_str^T[d][c] P[c][r]                (dV, DQ=false only)
// so P and dS feed the second MFMA straight from the accumulator registers, and the transposed
// streamed tiles are written to LDS in the matching key order (v_perm_b32 transposition in registers).
#include "mhip_common.hpp"

namespace mhip {
namespace {

constexpr int kD = 128;
constexpr int kTile = 64;             // streamed rows per main-loop tile
constexpr int kRowsPerWg = 128;       // stationary rows per workgroup (4 wavefronts x 32)
constexpr int kRmStride = kD + 8;     // row-major tile: bf16 per row (272 B)
constexpr int kTrStride = kTile + 8;  // transposed tile: bf16 per row (144 B)
constexpr int kRmBytes = kTile * kRmStride * 2;   // 17408
constexpr int kTrBytes = kD * kTrStride * 2;      // 18432
constexpr int kOffX = 0, kOffY = kRmBytes, kOffXT = 2 * kRmBytes, kOffYT = 2 * kRmBytes + kTrBytes;
constexpr int kOffLse = 2 * kRmBytes + 2 * kTrBytes, kOffDelta = kOffLse + kTile * 4;
constexpr int kSmemBytes = kOffDelta + kTile * 4;  // 72192
constexpr int kOStride = kD + 8;

struct BwdParams {
  const uint16_t* q; const uint16_t* k; const uint16_t* v; const uint16_t* dout;
  const float* lse; const float* delta;
  uint16_t* dq; uint16_t* dk; uint16_t* dv; float* dq_acc;
  int B, Sq, Sc, Hq, Hkv, group;
  int64_t q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, dk_sb, dk_ss, dk_sh;
  float scale, scale_log2;
  int n_tiles;      // stationary tiles per (batch, head)
  int total;
  int per_xcd;
  int heads_per_xcd;   // (batch, stationary head) pairs per XCD when they divide evenly, else 0
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

// delta = rowsum(dout * out): one row of 128 values per 16 lanes (8 values each)
__global__ __launch_bounds__(256) void bwd_delta(const uint16_t* __restrict__ dout, const uint16_t* __restrict__ out,
                                                 float* __restrict__ delta, int B, int Sq, int Hq,
                                                 int64_t sb, int64_t ss, int64_t sh) {
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int64_t rows = (int64_t)B * Hq * Sq;
  const int c = threadIdx.x & 15;
  float acc = 0.f;
  int b = 0, h = 0, s = 0;
  if (row < rows) {
    s = (int)(row % Sq);
    const int64_t bh = row / Sq;
    h = (int)(bh % Hq);
    b = (int)(bh / Hq);
    const int64_t off = b * sb + (int64_t)s * ss + h * sh + c * 8;
    const u32x4 a = *reinterpret_cast<const u32x4*>(dout + off);
    const u32x4 o = *reinterpret_cast<const u32x4*>(out + off);
#pragma unroll
    for (int j = 0; j < 4; ++j) acc += bf16_lo(a[j]) * bf16_lo(o[j]) + bf16_hi(a[j]) * bf16_hi(o[j]);
  }
#pragma unroll
  for (int m = 8; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 16);
  if (row < rows && c == 0) delta[row] = acc;      // (B, Hq, Sq) contiguous
}

template <bool DQ, bool CAUSAL>
__global__ __launch_bounds__(256, 1) void bwd_main(const BwdParams p) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[kSmemBytes];

  // Workgroup i runs on XCD i % 8: every XCD gets a contiguous range of (batch, head) pairs.  Under the
  // causal mask the work of a stationary tile grows (query tiles) or shrinks (key tiles) with its index:
  // such launches run the longest tiles first, across all heads.
  int st_tile, bh;
  if (!CAUSAL) {
    const int logical = (blockIdx.x & 7) * p.per_xcd + (blockIdx.x >> 3);
    if (logical >= p.total) return;
    st_tile = logical % p.n_tiles;
    bh = logical / p.n_tiles;
  } else {
    int rank;                                       // position in longest-first order
    if (p.heads_per_xcd > 0) {
      const int local = blockIdx.x >> 3;
      rank = local / p.heads_per_xcd;
      bh = (blockIdx.x & 7) * p.heads_per_xcd + local % p.heads_per_xcd;
    } else {
      if ((int)blockIdx.x >= p.total) return;
      const int nbh = p.total / p.n_tiles;
      rank = (int)blockIdx.x / nbh;
      bh = (int)blockIdx.x % nbh;
    }
    st_tile = DQ ? p.n_tiles - 1 - rank : rank;
  }
  const int hs = DQ ? bh % p.Hq : bh % p.Hkv;       // stationary head: a q head (DQ) or a kv head
  const int b = DQ ? bh / p.Hq : bh / p.Hkv;
  const int r0 = st_tile * kRowsPerWg;
  const int n_st = DQ ? p.Sq : p.Sc;                // stationary / streamed sequence lengths
  const int n_str = DQ ? p.Sc : p.Sq;
  const int shift = p.Sc - p.Sq;                    // causal: key j visible to query i iff j <= i + shift

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int ln = lane & 31;
  const int hf = lane >> 5;
  const int my_r = r0 + wave * 32 + ln;             // this lane's stationary row

  // ---- stationary operands: B operands of T1 / T2, lane (ln, hf) holds row[16 ks + 8 hf .. +7] -------
  bf16x8 xf[8], yf[8];
  {
    const int row = my_r < n_st ? my_r : n_st - 1;
    const uint16_t* xp; const uint16_t* yp;
    if (DQ) {
      const int64_t off = b * p.q_sb + (int64_t)row * p.q_ss + hs * p.q_sh + hf * 8;
      xp = p.q + off; yp = p.dout + off;
    } else {
      const int64_t off = b * p.k_sb + (int64_t)row * p.k_ss + hs * p.k_sh + hf * 8;
      xp = p.k + off; yp = p.v + off;
    }
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      xf[ks] = *reinterpret_cast<const bf16x8*>(xp + ks * 16);
      yf[ks] = *reinterpret_cast<const bf16x8*>(yp + ks * 16);
    }
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) { asm volatile("" : "+v"(xf[ks])); asm volatile("" : "+v"(yf[ks])); }
  }
  // DQ: the query is the stationary row, its lse / delta are per-lane scalars
  float lse2_lane = 0.f, delta_lane = 0.f;
  if (DQ) {
    const int row = my_r < n_st ? my_r : n_st - 1;
    const float l = p.lse[((int64_t)b * p.Hq + hs) * p.Sq + row];
    lse2_lane = (l == -INFINITY) ? INFINITY : l * kLog2e;     // rows that saw no key: P = 0
    delta_lane = p.delta[((int64_t)b * p.Hq + hs) * p.Sq + row];
  }

  // ---- streamed tiles ---------------------------------------------------------------------------------
  // DQ: K / V rows of kv head hs / group.  Otherwise: Q / dout rows of the `group` query heads that share
  // kv head hs, one head after the other.
  const int heads_str = DQ ? 1 : p.group;
  int first_tile = 0, tiles_per_head = (n_str + kTile - 1) / kTile;
  if (CAUSAL) {
    if (DQ) {   // keys beyond the last row's diagonal are hidden
      int lim = r0 + kRowsPerWg + shift;
      lim = lim < n_str ? lim : n_str;
      tiles_per_head = lim > 0 ? (lim + kTile - 1) / kTile : 0;
    } else {    // queries before the first key's diagonal see none of these keys
      const int i0 = r0 - shift;
      first_tile = i0 > 0 ? i0 / kTile : 0;
      if (first_tile > tiles_per_head) first_tile = tiles_per_head;
    }
  }
  const int span = tiles_per_head - first_tile;
  const int ntiles = span * heads_str;

  const int ld_chunk = tid & 15;
  const int ld_quad = tid >> 4;                       // rows 4 quad .. 4 quad + 3 of the tile
  const uint16_t* xbase; const uint16_t* ybase; int64_t s_ss, s_sh; uint32_t s_bytes;
  if (DQ) {
    const int hk = hs / p.group;
    xbase = p.k + b * p.k_sb + hk * p.k_sh; ybase = p.v + b * p.k_sb + hk * p.k_sh;
    s_ss = p.k_ss; s_sh = 0;
    s_bytes = (uint32_t)(((int64_t)(p.Sc - 1) * p.k_ss + kD) * 2);
  } else {
    xbase = p.q + b * p.q_sb; ybase = p.dout + b * p.q_sb;
    s_ss = p.q_ss; s_sh = p.q_sh;
    s_bytes = (uint32_t)(((int64_t)(p.Sq - 1) * p.q_ss + (int64_t)(p.Hq - 1) * p.q_sh + kD) * 2);
  }
  const __amdgpu_buffer_rsrc_t xrs = make_rsrc(xbase, s_bytes);
  const __amdgpu_buffer_rsrc_t yrs = make_rsrc(ybase, s_bytes);
  int goff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) goff[i] = (int)((ld_quad * 4 + i) * s_ss * 2) + ld_chunk * 16;
  u32x4 xreg[4], yreg[4];
  float lse_reg = 0.f, delta_reg = 0.f;

  // tile index -> (head of the group, first streamed row)
  auto tile_head = [&](int t) { return DQ ? 0 : t / span; };
  auto tile_row0 = [&](int t) { return (first_tile + (DQ ? t : t % span)) * kTile; };

  auto load_tile = [&](int t) {
    const int hq = DQ ? 0 : hs * p.group + tile_head(t);
    const int c0 = tile_row0(t);
    const int soff = (int)(((int64_t)c0 * s_ss + (int64_t)hq * s_sh) * 2);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      xreg[i] = __builtin_amdgcn_raw_buffer_load_b128(xrs, goff[i], soff, 0);
      yreg[i] = __builtin_amdgcn_raw_buffer_load_b128(yrs, goff[i], soff, 0);
    }
    if (!DQ && tid < kTile) {
      const int i = c0 + tid;
      if (i < p.Sq) {
        const float l = p.lse[((int64_t)b * p.Hq + hq) * p.Sq + i];
        lse_reg = (l == -INFINITY) ? INFINITY : l * kLog2e;
        delta_reg = p.delta[((int64_t)b * p.Hq + hq) * p.Sq + i];
      } else {
        lse_reg = INFINITY;     // rows past the end of the shard: P = 0
        delta_reg = 0.f;
      }
    }
  };

  // transposed tiles use the layout of V^T in the forward kernel: row d of the tile lives in LDS row
  // d ^ rev3(d >> 4), and inside a row the streamed rows are ordered the way the accumulator registers
  // of one MFMA k-step hold them
  const int tr_off = ((ld_quad >> 2) * 2 + (ld_quad & 1)) * 16 + ((ld_quad & 3) >> 1) * 8;
  const int tr_xor = ((ld_chunk >> 3) & 1) | (((ld_chunk >> 2) & 1) << 1) | (((ld_chunk >> 1) & 1) << 2);
  auto store_transposed = [&](unsigned char* dst, const u32x4 (&reg)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      u32x2 even, odd;
      even[0] = __builtin_amdgcn_perm(reg[1][j], reg[0][j], 0x05040100u);
      even[1] = __builtin_amdgcn_perm(reg[3][j], reg[2][j], 0x05040100u);
      odd[0] = __builtin_amdgcn_perm(reg[1][j], reg[0][j], 0x07060302u);
      odd[1] = __builtin_amdgcn_perm(reg[3][j], reg[2][j], 0x07060302u);
      const int r_even = ld_chunk * 8 + ((2 * j) ^ tr_xor);
      const int r_odd = ld_chunk * 8 + ((2 * j + 1) ^ tr_xor);
      *reinterpret_cast<u32x2*>(dst + r_even * (kTrStride * 2) + tr_off) = even;
      *reinterpret_cast<u32x2*>(dst + r_odd * (kTrStride * 2) + tr_off) = odd;
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int off = (ld_quad * 4 + i) * (kRmStride * 2) + ld_chunk * 16;
      *reinterpret_cast<u32x4*>(smem + kOffX + off) = xreg[i];
      *reinterpret_cast<u32x4*>(smem + kOffY + off) = yreg[i];
    }
    store_transposed(smem + kOffXT, xreg);
    if (!DQ) {
      store_transposed(smem + kOffYT, yreg);
      if (tid < kTile) {
        reinterpret_cast<float*>(smem + kOffLse)[tid] = lse_reg;
        reinterpret_cast<float*>(smem + kOffDelta)[tid] = delta_reg;
      }
    }
  };

  const int rm_rd = ln * (kRmStride * 2) + hf * 16;      // + mb*32*272 + kk*32
  int tr_rd[4];                                            // + kstep*32
#pragma unroll
  for (int db = 0; db < 4; ++db) {
    const int x = (db >> 1) | ((db & 1) << 1) | ((ln >> 4) << 2);
    tr_rd[db] = (db * 32 + (ln ^ x)) * (kTrStride * 2) + hf * 16;
  }

  f32x16 acc1[4], acc2[4];      // DQ: acc1 = dQ^T.  Otherwise acc1 = dK^T, acc2 = dV^T
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) { acc1[i][j] = 0.f; acc2[i][j] = 0.f; }
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  if (ntiles > 0) load_tile(0);
  for (int t = 0; t < ntiles; ++t) {
    __syncthreads();                 // everybody is done reading the previous tile
    store_tile();
    if (t + 1 < ntiles) load_tile(t + 1);
    __syncthreads();

    // ---- T1 = X_str X_st^T (scores), T2 = Y_str Y_st^T (dP): 64 streamed x 32 stationary rows ----------
    f32x16 t1[2], t2[2];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        const int off = rm_rd + mb * (32 * kRmStride * 2) + kk * 32;
        const bf16x8 xa = *reinterpret_cast<const bf16x8*>(smem + kOffX + off);
        const bf16x8 ya = *reinterpret_cast<const bf16x8*>(smem + kOffY + off);
        t1[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa, xf[kk], kk == 0 ? zero : t1[mb], 0, 0, 0);
        t2[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ya, yf[kk], kk == 0 ? zero : t2[mb], 0, 0, 0);
      }
    }

    // ---- P = exp2(scale_log2 T1 - lse log2e), dS = P (T2 - delta), hidden elements -> 0 ----------------
    const int c0 = tile_row0(t);
    bf16x8 pfrag[4], dsfrag[4];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      float pv[16], dsv[16];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float l4[4], d4[4];
        if (DQ) {
#pragma unroll
          for (int e = 0; e < 4; ++e) { l4[e] = lse2_lane; d4[e] = delta_lane; }
        } else {
          const int row = mb * 32 + g * 8 + hf * 4;
          const f32x4 lv = *reinterpret_cast<const f32x4*>(smem + kOffLse + row * 4);
          const f32x4 dv = *reinterpret_cast<const f32x4*>(smem + kOffDelta + row * 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) { l4[e] = lv[e]; d4[e] = dv[e]; }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int j = g * 4 + e;
          const int c = c0 + mb * 32 + g * 8 + hf * 4 + e;       // streamed row of this element
          float pe = fast_exp2(__builtin_fmaf(t1[mb][j], p.scale_log2, -l4[e]));
          bool hidden = DQ ? (c >= p.Sc) : false;                 // keys past the chunk (zero filled)
          if (CAUSAL) hidden = hidden || (DQ ? (c > my_r + shift) : (my_r > c + shift));
          if (hidden) pe = 0.f;
          pv[j] = pe;
          dsv[j] = pe * (t2[mb][j] - d4[e]);
        }
      }
#pragma unroll
      for (int j2 = 0; j2 < 2; ++j2) {
        u32x4 wp, wd;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          wp[e] = pack_bf16(pv[8 * j2 + 2 * e], pv[8 * j2 + 2 * e + 1]);
          wd[e] = pack_bf16(dsv[8 * j2 + 2 * e], dsv[8 * j2 + 2 * e + 1]);
        }
        pfrag[mb * 2 + j2] = __builtin_bit_cast(bf16x8, wp);
        dsfrag[mb * 2 + j2] = __builtin_bit_cast(bf16x8, wd);
      }
    }

    // ---- acc1^T += X_str^T dS,  acc2^T += Y_str^T P ------------------------------------------------------
#pragma unroll
    for (int kstep = 0; kstep < 4; ++kstep) {
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const bf16x8 xt = *reinterpret_cast<const bf16x8*>(smem + kOffXT + tr_rd[db] + kstep * 32);
        acc1[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xt, dsfrag[kstep], acc1[db], 0, 0, 0);
        if (!DQ) {
          const bf16x8 yt = *reinterpret_cast<const bf16x8*>(smem + kOffYT + tr_rd[db] + kstep * 32);
          acc2[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(yt, pfrag[kstep], acc2[db], 0, 0, 0);
        }
      }
    }
  }

  // ---- epilogue: acc^T[d][r] -> rows of the output through LDS --------------------------------------------
  auto write_out = [&](const f32x16 (&acc)[4], float mul, uint16_t* dst, int64_t d_sb, int64_t d_ss,
                       int64_t d_sh, int head) {
    __syncthreads();
    unsigned char* os = smem + wave * (32 * kOStride * 2);
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        w[0] = pack_bf16(acc[db][4 * g] * mul, acc[db][4 * g + 1] * mul);
        w[1] = pack_bf16(acc[db][4 * g + 2] * mul, acc[db][4 * g + 3] * mul);
        *reinterpret_cast<u32x2*>(os + ln * (kOStride * 2) + (db * 32 + g * 8 + hf * 4) * 2) = w;
      }
    __syncthreads();
    const int chunk = lane & 15;
    uint16_t* op = dst + b * d_sb + head * d_sh + chunk * 8;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int r = (lane >> 4) + 4 * it;
      const int row = r0 + wave * 32 + r;
      if (row < n_st) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(os + r * (kOStride * 2) + chunk * 16);
        *reinterpret_cast<u32x4*>(op + (int64_t)row * d_ss) = w;
      }
    }
  };
  if (DQ) {
    write_out(acc1, p.scale, p.dq, p.q_sb, p.q_ss, p.q_sh, hs);
    if (p.dq_acc != nullptr && my_r < n_st) {
      // fp32 accumulator (B, Sq, Hq, D) contiguous; every element belongs to exactly one lane
      float* ap = p.dq_acc + (((int64_t)b * p.Sq + my_r) * p.Hq + hs) * kD;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x4* a4 = reinterpret_cast<f32x4*>(ap + db * 32 + g * 8 + hf * 4);
          f32x4 v = *a4;
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += acc1[db][4 * g + e] * p.scale;
          *a4 = v;
        }
    }
  } else {
    write_out(acc1, p.scale, p.dk, p.dk_sb, p.dk_ss, p.dk_sh, hs);
    write_out(acc2, 1.f, p.dv, p.dk_sb, p.dk_ss, p.dk_sh, hs);
  }
}

}  // namespace
}  // namespace mhip

using namespace mhip;

extern "C" int64_t mhip_attn_bwd_workspace_bytes(int B, int Sq, int Sc, int Hq, int Hkv, int D) {
  (void)Sc; (void)Hkv; (void)D;
  if (B < 0 || Sq < 0 || Hq < 0) return 0;
  return (int64_t)B * Hq * Sq * 4 + 16;     // delta (B, Hq, Sq) fp32
}

extern "C" int mhip_attn_bwd_block(const void* dout, const void* q, const void* k, const void* v,
                                   const void* out, const float* lse,
                                   void* dq, void* dk, void* dv, float* dq_acc,
                                   int B, int Sq, int Sc, int Hq, int Hkv, int D,
                                   int64_t q_sb, int64_t q_ss, int64_t q_sh,
                                   int64_t k_sb, int64_t k_ss, int64_t k_sh,
                                   int64_t dk_sb, int64_t dk_ss, int64_t dk_sh,
                                   float softmax_scale, int mask, int deterministic,
                                   void* workspace, void* stream) {
  (void)deterministic;   // there are no atomics: every run is deterministic
  if (B < 0 || Sq < 0 || Sc < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return MHIP_EINVAL;
  if (!(softmax_scale > 0.f) || !(softmax_scale < INFINITY)) return MHIP_EINVAL;
  if (mask != MHIP_MASK_NONE && mask != MHIP_MASK_CAUSAL) return MHIP_EINVAL;
  if (D != kD) return MHIP_EHEADDIM;
  if (B == 0) return MHIP_OK;
  if (Sq > 0 && (!dout || !q || !out || !lse || !dq || !workspace)) return MHIP_EINVAL;
  if (Sc > 0 && (!k || !v || !dk || !dv)) return MHIP_EINVAL;
  const void* ptrs[] = {dout, q, k, v, out, dq, dk, dv, workspace, dq_acc};
  for (const void* ptr : ptrs)
    if (ptr && !aligned16(ptr)) return MHIP_EALIGN;
  const int64_t strides[] = {q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, dk_sb, dk_ss, dk_sh};
  for (int64_t s : strides)
    if (s < 0 || (s & 7)) return MHIP_EALIGN;
  // streamed tiles are fetched through 32-bit buffer offsets
  const int64_t q_span = ((int64_t)Sq * q_ss + (int64_t)Hq * q_sh) * 2;
  const int64_t k_span = (int64_t)Sc * k_ss * 2;
  if (q_span >= (int64_t(1) << 31) || k_span >= (int64_t(1) << 31)) return MHIP_EUNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);

  BwdParams p;
  p.q = static_cast<const uint16_t*>(q); p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v); p.dout = static_cast<const uint16_t*>(dout);
  p.lse = lse; p.delta = static_cast<const float*>(workspace);
  p.dq = static_cast<uint16_t*>(dq); p.dk = static_cast<uint16_t*>(dk); p.dv = static_cast<uint16_t*>(dv);
  p.dq_acc = dq_acc;
  p.B = B; p.Sq = Sq; p.Sc = Sc; p.Hq = Hq; p.Hkv = Hkv; p.group = Hq / Hkv;
  p.q_sb = q_sb; p.q_ss = q_ss; p.q_sh = q_sh;
  p.k_sb = k_sb; p.k_ss = k_ss; p.k_sh = k_sh;
  p.dk_sb = dk_sb; p.dk_ss = dk_ss; p.dk_sh = dk_sh;
  p.scale = softmax_scale; p.scale_log2 = softmax_scale * kLog2e;
  const bool causal = mask == MHIP_MASK_CAUSAL;

  if (Sq > 0) {
    const int64_t rows = (int64_t)B * Hq * Sq;
    hipLaunchKernelGGL(bwd_delta, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, st,
                       static_cast<const uint16_t*>(dout), static_cast<const uint16_t*>(out),
                       static_cast<float*>(workspace), B, Sq, Hq, q_sb, q_ss, q_sh);
    // dQ: one workgroup per 128 query rows
    p.n_tiles = (Sq + kRowsPerWg - 1) / kRowsPerWg;
    p.total = B * Hq * p.n_tiles;
    p.per_xcd = (p.total + 7) / 8;
    p.heads_per_xcd = (B * Hq) % 8 == 0 ? (B * Hq) / 8 : 0;
    if (causal) hipLaunchKernelGGL((bwd_main<true, true>), dim3(p.per_xcd * 8), dim3(256), 0, st, p);
    else hipLaunchKernelGGL((bwd_main<true, false>), dim3(p.per_xcd * 8), dim3(256), 0, st, p);
  }
  if (Sc > 0) {
    // dK, dV: one workgroup per 128 keys of one kv head
    p.n_tiles = (Sc + kRowsPerWg - 1) / kRowsPerWg;
    p.total = B * Hkv * p.n_tiles;
    p.per_xcd = (p.total + 7) / 8;
    p.heads_per_xcd = (B * Hkv) % 8 == 0 ? (B * Hkv) / 8 : 0;
    if (causal) hipLaunchKernelGGL((bwd_main<false, true>), dim3(p.per_xcd * 8), dim3(256), 0, st, p);
    else hipLaunchKernelGGL((bwd_main<false, false>), dim3(p.per_xcd * 8), dim3(256), 0, st, p);
  }
  return launch_status();
}
