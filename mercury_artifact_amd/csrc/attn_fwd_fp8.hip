// Block forward on e4m3 (OCP float8) Q/K/V for gfx950: out = softmax(scale * q k^T) v in bf16 and
// lse in fp32, with x ~ descale_x * x_q per tensor.  fp8 MFMA (v_mfma_f32_32x32x16_fp8_fp8) for both
// contractions, fp32 softmax.  Not in the reference; same call boundary as the bf16 kernel
// (utils/flash_attn_dsl.py:159-176) with three extra descale arguments.
//
// Same decomposition as the bf16 kernel: 8 wavefronts x 32 Q rows per workgroup, wavefronts 0-3 stage K
// and 4-7 stage V^T, S^T = K Q^T keeps one Q row per lane, P^T feeds the second MFMA from the
// accumulator registers.  Differences:
//   * a main-loop tile is 128 keys (the tile is as many bytes as the 64-key bf16 tile);
//   * one 16-byte LDS read carries the A operands of two MFMA k-steps (8 fp8 values each);
//   * the descales fold into the softmax scale (q, k) and the final normalisation (v);
//   * P is multiplied by 2^7 before it is rounded to e4m3 (and the result divided by 2^7), so that small
//     probabilities keep their relative precision; the reference score only lags the running maximum by
//     at most one binade, which keeps 2^7 P below the e4m3 maximum of 448.
#include "mhip_common.hpp"

namespace mhip {
namespace {

constexpr int kD = 128;
constexpr int kWaves = 8;
constexpr int kBM = kWaves * 32;
constexpr int kBN = 128;              // keys per tile
constexpr int kStride = 128 + 16;     // bytes per LDS row of K (128 head-dim bytes) and of V^T (128 keys)
constexpr int kTileBytes = 128 * kStride;          // 18432, K and V^T alike
constexpr int kStageBytes = 2 * kTileBytes;
constexpr int kOStride = kD + 8;
constexpr float kPShift = 7.f;        // P is stored as 2^7 P in e4m3
constexpr float kRescaleSlack = 1.f;

struct Fp8Params {
  const uint8_t* q; const uint8_t* k; const uint8_t* v;
  uint16_t* out; float* lse;
  int B, Sq, Sc, Hq, Hkv, group;
  int64_t q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, v_sb, v_ss, v_sh, o_sb, o_ss, o_sh;
  float scale_eff;       // softmax_scale * q_descale * k_descale: natural-log scale of the integer-like dot
  float scale_log2;      // scale_eff * log2(e)
  float out_mul;         // v_descale
  int nq_tiles, total, per_xcd, heads_per_xcd;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ long as_long(uint32_t lo, uint32_t hi) {
  return (long)(((unsigned long)hi << 32) | lo);
}

template <bool CAUSAL>
__global__ __launch_bounds__(kWaves * 64, 2) void attn_fwd_fp8_d128(const Fp8Params p) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * kStageBytes];

  // Workgroup i runs on XCD i % 8: every XCD gets a contiguous range of (batch, head) pairs, so the
  // workgroups that share a K/V head share an L2.  Causal launches run the longest Q tiles first,
  // across all heads.
  int qt, bh;
  if (!CAUSAL) {
    const int logical = (blockIdx.x & 7) * p.per_xcd + (blockIdx.x >> 3);
    if (logical >= p.total) return;
    qt = logical % p.nq_tiles;
    bh = logical / p.nq_tiles;
  } else if (p.heads_per_xcd > 0) {
    const int local = blockIdx.x >> 3;
    qt = p.nq_tiles - 1 - local / p.heads_per_xcd;
    bh = (blockIdx.x & 7) * p.heads_per_xcd + local % p.heads_per_xcd;
  } else {
    if ((int)blockIdx.x >= p.total) return;
    const int nbh = p.B * p.Hq;
    qt = p.nq_tiles - 1 - (int)blockIdx.x / nbh;
    bh = (int)blockIdx.x % nbh;
  }
  const int hq = bh % p.Hq;
  const int b = bh / p.Hq;
  const int hk = hq / p.group;
  const int q0 = qt * kBM;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int ln = lane & 31;
  const int hf = lane >> 5;
  const bool v_loader = wave >= 4;

  int kv_end = p.Sc;
  if (CAUSAL) {
    const int lim = q0 + kBM + (p.Sc - p.Sq);
    kv_end = lim < kv_end ? lim : kv_end;
    if (kv_end < 0) kv_end = 0;
  }
  const int ntiles = (kv_end + kBN - 1) / kBN;

  // ---- Q fragment: lane (ln, hf) holds bytes [32 i + 16 hf, +16) of its row; the first 8 are the B
  // operand of k-step 2i, the last 8 of k-step 2i+1 (K is read from LDS with the same split) ------------
  const int my_q = q0 + wave * 32 + ln;
  u32x4 qf[4];
  {
    const int row = my_q < p.Sq ? my_q : p.Sq - 1;
    const uint8_t* qp = p.q + b * p.q_sb + (int64_t)row * p.q_ss + hq * p.q_sh + hf * 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) qf[i] = *reinterpret_cast<const u32x4*>(qp + i * 32);
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(qf[i]));
  }

  // ---- staging: K loader thread lt loads rows (lt/8 + 32 i), 16-byte chunk lt%8; V loader thread loads
  // the four rows of key quad lt/8, chunk lt%8 (16 head-dim values each) ---------------------------------
  const int lt = tid & 255;
  const int ld_chunk = lt & 7;
  const int ld_row = lt >> 3;                        // 0..31
  const uint8_t* gbase = v_loader ? p.v + b * p.v_sb + hk * p.v_sh : p.k + b * p.k_sb + hk * p.k_sh;
  const int64_t g_ss = v_loader ? p.v_ss : p.k_ss;
  const __amdgpu_buffer_rsrc_t grs = make_rsrc(gbase, (uint32_t)((int64_t)(p.Sc - 1) * g_ss + kD));
  int goff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    goff[i] = (int)((v_loader ? ld_row * 4 + i : ld_row + 32 * i) * g_ss) + ld_chunk * 16;
  const int tile_bytes = (int)(kBN * g_ss);
  u32x4 greg[4];
  auto load_tile = [&](int t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) greg[i] = __builtin_amdgcn_raw_buffer_load_b128(grs, goff[i], t * tile_bytes, 0);
  };

  // V^T row d lives in LDS row d ^ ((d >> 4) & 7); inside a row, key quad (4 keys) u = 4-key index:
  // 32-key block mb = u / 8, then (jj, thi, hf) = bits 2, 1, 0 of u % 8 -> byte (2 mb + hf) 16 + 8 jj + 4 thi,
  // which is the order the accumulator registers of S^T hold the keys of two consecutive MFMA k-steps.
  const int vt_off = ((ld_row >> 3) * 2 + (ld_row & 1)) * 16 + ((ld_row >> 2) & 1) * 8 + ((ld_row >> 1) & 1) * 4;
  auto store_tile = [&](int stage) {
    if (!v_loader) {
      unsigned char* ks = smem + stage * kStageBytes;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<u32x4*>(ks + (ld_row + 32 * i) * kStride + ld_chunk * 16) = greg[i];
    } else {
      unsigned char* vs = smem + stage * kStageBytes + kTileBytes;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        // dword w of each of the four rows holds head-dim values 4w .. 4w+3 of this chunk
        const uint32_t t01_lo = __builtin_amdgcn_perm(greg[1][w], greg[0][w], 0x05010400u);   // d0:(k0,k1) d1:(k0,k1)
        const uint32_t t01_hi = __builtin_amdgcn_perm(greg[1][w], greg[0][w], 0x07030602u);   // d2, d3
        const uint32_t t23_lo = __builtin_amdgcn_perm(greg[3][w], greg[2][w], 0x05010400u);
        const uint32_t t23_hi = __builtin_amdgcn_perm(greg[3][w], greg[2][w], 0x07030602u);
        uint32_t o[4];
        o[0] = __builtin_amdgcn_perm(t23_lo, t01_lo, 0x05040100u);
        o[1] = __builtin_amdgcn_perm(t23_lo, t01_lo, 0x07060302u);
        o[2] = __builtin_amdgcn_perm(t23_hi, t01_hi, 0x05040100u);
        o[3] = __builtin_amdgcn_perm(t23_hi, t01_hi, 0x07060302u);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int d = ld_chunk * 16 + ((4 * w + e) ^ ld_chunk);
          *reinterpret_cast<uint32_t*>(vs + d * kStride + vt_off) = o[e];
        }
      }
    }
  };

  const int k_rd = ln * kStride + hf * 16;            // + mb*32*144 + i*32
  int v_rd[4];                                         // + (2 mb) * 16
#pragma unroll
  for (int db = 0; db < 4; ++db) {
    const int x = (db * 2 + (ln >> 4)) & 7;            // (d >> 4) & 7 for d = 32 db + ln
    v_rd[db] = (db * 32 + (ln ^ x)) * kStride + hf * 16;
  }
  const int causal_shift = p.Sc - p.Sq;

  f32x16 o_acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) o_acc[i][j] = 0.f;
  float m_ref = -INFINITY, l_run = 0.f;      // l_run sums 2^7 P (this lane's half of the keys)
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  if (ntiles > 0) {
    load_tile(0);
    store_tile(0);
  }
  for (int t = 0; t < ntiles; ++t) {
    const int stage = t & 1;
    if (t + 1 < ntiles) load_tile(t + 1);
    __syncthreads();
    const unsigned char* ks = smem + stage * kStageBytes;
    const unsigned char* vs = ks + kTileBytes;

    // ---- S^T tile: 128 keys x 32 q rows per wave ------------------------------------------------------
    f32x16 s[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) {
        const u32x4 kf = *reinterpret_cast<const u32x4*>(ks + k_rd + mb * (32 * kStride) + i * 32);
        s[mb] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(as_long(kf[0], kf[1]), as_long(qf[i][0], qf[i][1]),
                                                           i == 0 ? zero : s[mb], 0, 0, 0);
        s[mb] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(as_long(kf[2], kf[3]), as_long(qf[i][2], qf[i][3]),
                                                           s[mb], 0, 0, 0);
      }
    }

    const int kv0 = t * kBN;
    bool need_mask = kv0 + kBN > p.Sc;
    if (CAUSAL) need_mask = need_mask || (kv0 + kBN - 1 > q0 + causal_shift);
    if (need_mask) {
      int lim = p.Sc - 1;
      if (CAUSAL) { const int c = my_q + causal_shift; lim = c < lim ? c : lim; }
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int key = kv0 + mb * 32 + (j >> 2) * 8 + hf * 4 + (j & 3);
          if (key > lim) s[mb][j] = -INFINITY;
        }
    }

    // ---- online softmax ------------------------------------------------------------------------------------
    float mx = s[0][0];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int j = 0; j < 16; ++j) mx = fmaxf(mx, s[mb][j]);
    mx = pair_max(mx);
    const bool grow = (mx - m_ref) * p.scale_log2 > kRescaleSlack;
    if (__builtin_amdgcn_ballot_w64(grow) != 0) {
      const float m_new = grow ? mx : m_ref;
      const float alpha = (m_new == -INFINITY) ? 1.f : fast_exp2((m_ref - m_new) * p.scale_log2);
      m_ref = m_new;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int j = 0; j < 16; ++j) o_acc[db][j] *= alpha;
    }
    const float msc = (m_ref == -INFINITY) ? 0.f : m_ref * p.scale_log2 - kPShift;   // exponent of 2^7 P
    float rs = 0.f;
    u32x4 pf[4];               // pf[mb]: dwords 0,1 = k-step (mb, 0), dwords 2,3 = k-step (mb, 1)
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float e = fast_exp2(__builtin_fmaf(s[mb][j], p.scale_log2, -msc));
        rs += e;
        s[mb][j] = e;
      }
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        int packed = 0;
        packed = __builtin_amdgcn_cvt_pk_fp8_f32(s[mb][4 * w], s[mb][4 * w + 1], packed, false);
        packed = __builtin_amdgcn_cvt_pk_fp8_f32(s[mb][4 * w + 2], s[mb][4 * w + 3], packed, true);
        pf[mb][w] = (uint32_t)packed;
      }
    }
    l_run += rs;

    // ---- O^T += V^T P^T -----------------------------------------------------------------------------------
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const u32x4 vf = *reinterpret_cast<const u32x4*>(vs + v_rd[db] + mb * 32);
        o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(as_long(vf[0], vf[1]), as_long(pf[mb][0], pf[mb][1]),
                                                               o_acc[db], 0, 0, 0);
        o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(as_long(vf[2], vf[3]), as_long(pf[mb][2], pf[mb][3]),
                                                               o_acc[db], 0, 0, 0);
      }
    }

    if (t + 1 < ntiles) store_tile(stage ^ 1);
  }

  // ---- epilogue ---------------------------------------------------------------------------------------------
  const float l_tot = pair_sum(l_run);
  const float inv = l_tot > 0.f ? p.out_mul / l_tot : 0.f;           // the two factors 2^7 cancel
  if (hf == 0 && my_q < p.Sq) {
    const float lse = l_tot > 0.f ? m_ref * p.scale_eff + (fast_log2(l_tot) - kPShift) * kLn2 : -INFINITY;
    p.lse[((int64_t)b * p.Hq + hq) * p.Sq + my_q] = lse;
  }
  __syncthreads();
  unsigned char* os = smem + wave * (32 * kOStride * 2);
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w;
      w[0] = pack_bf16(o_acc[db][4 * g] * inv, o_acc[db][4 * g + 1] * inv);
      w[1] = pack_bf16(o_acc[db][4 * g + 2] * inv, o_acc[db][4 * g + 3] * inv);
      *reinterpret_cast<u32x2*>(os + ln * (kOStride * 2) + (db * 32 + g * 8 + hf * 4) * 2) = w;
    }
  __syncthreads();
  {
    const int chunk = lane & 15;
    uint16_t* op = p.out + b * p.o_sb + hq * p.o_sh + chunk * 8;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int r = (lane >> 4) + 4 * it;
      const int row = q0 + wave * 32 + r;
      if (row < p.Sq) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(os + r * (kOStride * 2) + chunk * 16);
        *reinterpret_cast<u32x4*>(op + (int64_t)row * p.o_ss) = w;
      }
    }
  }
}

}  // namespace

int attn_fwd_fp8(const void* q, const void* k, const void* v, void* out, float* lse,
                 int B, int Sq, int Sc, int Hq, int Hkv, const int64_t* st, float scale, int mask,
                 float q_descale, float k_descale, float v_descale, hipStream_t stream) {
  Fp8Params p;
  p.q = static_cast<const uint8_t*>(q); p.k = static_cast<const uint8_t*>(k); p.v = static_cast<const uint8_t*>(v);
  p.out = static_cast<uint16_t*>(out); p.lse = lse;
  p.B = B; p.Sq = Sq; p.Sc = Sc; p.Hq = Hq; p.Hkv = Hkv; p.group = Hq / Hkv;
  p.q_sb = st[0]; p.q_ss = st[1]; p.q_sh = st[2];
  p.k_sb = st[3]; p.k_ss = st[4]; p.k_sh = st[5];
  p.v_sb = st[6]; p.v_ss = st[7]; p.v_sh = st[8];
  p.o_sb = st[9]; p.o_ss = st[10]; p.o_sh = st[11];
  p.scale_eff = scale * q_descale * k_descale;
  p.scale_log2 = p.scale_eff * kLog2e;
  p.out_mul = v_descale;
  p.nq_tiles = (Sq + kBM - 1) / kBM;
  p.total = B * Hq * p.nq_tiles;
  p.per_xcd = (p.total + 7) / 8;
  p.heads_per_xcd = (B * Hq) % 8 == 0 ? (B * Hq) / 8 : 0;
  const dim3 grid(p.per_xcd * 8), block(kWaves * 64);
  if (mask == MHIP_MASK_CAUSAL) hipLaunchKernelGGL(attn_fwd_fp8_d128<true>, grid, block, 0, stream, p);
  else hipLaunchKernelGGL(attn_fwd_fp8_d128<false>, grid, block, 0, stream, p);
  return launch_status();
}

}  // namespace mhip
