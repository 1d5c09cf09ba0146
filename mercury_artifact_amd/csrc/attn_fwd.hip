// Block forward of the ring-attention step for gfx950: one Q shard against one KV chunk,
// out = softmax(scale * q k^T) v and lse = logsumexp(scale * q k^T), bf16 in, fp32 accumulate.
//
// Replaces the flash-attn call at utils/flash_attn_dsl.py:159-176 of the reference.
//
// Work decomposition
//   workgroup  = 128 Q rows of one (batch, q-head): 4 wavefronts x 32 rows, two workgroups per CU
//   main loop  = 64-key tiles of the chunk, K and V double-buffered in LDS
//   S^T = K Q^T  : v_mfma_f32_32x32x16_bf16 with A = K rows (LDS), B = Q (registers, loaded once).
//                  The accumulator layout puts one Q row in each lane (lane % 32) and 32 of the
//                  64 keys of the tile in that lane's registers, so the online softmax needs one
//                  exchange with lane ^ 32 per tile and no other cross-lane traffic.
//   O^T = V^T P^T: the same lane that produced P^T[key][q] feeds it back as the B operand; the
//                  key order inside one MFMA k-step is whatever the accumulator registers hold,
//                  and V^T is written to LDS in exactly that key order, so P never moves.
//   V^T          : transposed in registers (v_perm_b32) on its way from global memory to LDS.
#include "mhip_common.hpp"

namespace mhip {
namespace {

constexpr int kD = 128;            // head dimension
constexpr int kBM = 128;           // Q rows per workgroup
constexpr int kBN = 64;            // keys per main-loop tile
constexpr int kThreads = 256;
constexpr int kKStride = kD + 8;   // bf16 elements per K row in LDS (272 B: 16 B skew per row)
constexpr int kVStride = kBN + 8;  // bf16 elements per V^T row in LDS (144 B)
constexpr int kKBytes = kBN * kKStride * 2;   // 17408
constexpr int kVBytes = kD * kVStride * 2;    // 18432
constexpr int kStageBytes = kKBytes + kVBytes;
constexpr int kOStride = kD + 8;   // epilogue staging of O, bf16 elements per row

struct FwdParams {
  const uint16_t* q; const uint16_t* k; const uint16_t* v;
  uint16_t* out; float* lse;
  int B, Sq, Sc, Hq, Hkv, group;
  int64_t q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, v_sb, v_ss, v_sh, o_sb, o_ss, o_sh;
  float scale, scale_log2;
  int nq_tiles;      // ceil(Sq / 128)
  int total;         // B * Hq * nq_tiles
  int per_xcd;       // ceil(total / 8)
};

template <bool CAUSAL>
__global__ __launch_bounds__(kThreads, 2) void attn_fwd_bf16_d128(const FwdParams p) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * kStageBytes];

  // Workgroup i runs on XCD i % 8.  Give every XCD a contiguous range of the (batch, head, q-tile)
  // order so that the workgroups sharing one K/V head also share one L2.
  const int logical = (blockIdx.x & 7) * p.per_xcd + (blockIdx.x >> 3);
  if (logical >= p.total) return;
  int qt = logical % p.nq_tiles;
  const int bh = logical / p.nq_tiles;
  const int hq = bh % p.Hq;
  const int b = bh / p.Hq;
  const int hk = hq / p.group;
  if (CAUSAL) qt = p.nq_tiles - 1 - qt;          // longest rows first
  const int q0 = qt * kBM;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int ln = lane & 31;
  const int hf = lane >> 5;

  // ---- number of key tiles this Q tile has to visit -------------------------------------------
  int kv_end = p.Sc;
  if (CAUSAL) {
    const int lim = q0 + kBM + (p.Sc - p.Sq);     // one past the last key visible to the last row
    kv_end = lim < kv_end ? lim : kv_end;
    if (kv_end < 0) kv_end = 0;
  }
  const int ntiles = (kv_end + kBN - 1) / kBN;

  // ---- Q fragment: B operand of S^T = K Q^T, lane (ln, hf) holds Q[row][16 ks + 8 hf .. +7] -----
  const int my_q = q0 + wave * 32 + ln;
  bf16x8 qf[8];
  {
    const int row = my_q < p.Sq ? my_q : p.Sq - 1;
    const uint16_t* qp = p.q + b * p.q_sb + (int64_t)row * p.q_ss + hq * p.q_sh + hf * 8;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + ks * 16);
  }

  // ---- global -> register staging of one K/V tile ---------------------------------------------
  // K: thread loads rows (tid/16 + 16 i), 16-byte chunk tid%16.
  // V: thread loads the four rows of key quad tid/16, chunk tid%16 (8 head-dim values each).
  const int ld_chunk = tid & 15;
  const int ld_row = tid >> 4;
  const uint16_t* kbase = p.k + b * p.k_sb + hk * p.k_sh + ld_chunk * 8;
  const uint16_t* vbase = p.v + b * p.v_sb + hk * p.v_sh + ld_chunk * 8;
  u32x4 kreg[4], vreg[4];

  auto load_tile = [&](int t) {
    const int kv0 = t * kBN;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int rk = kv0 + ld_row + 16 * i;
      rk = rk < p.Sc ? rk : p.Sc - 1;
      kreg[i] = *reinterpret_cast<const u32x4*>(kbase + (int64_t)rk * p.k_ss);
      int rv = kv0 + ld_row * 4 + i;
      rv = rv < p.Sc ? rv : p.Sc - 1;
      vreg[i] = *reinterpret_cast<const u32x4*>(vbase + (int64_t)rv * p.v_ss);
    }
  };

  // LDS position of key quad (4 consecutive keys) inside a V^T row: MFMA k-step = quad / 4,
  // lane half = quad % 2, first / second group of four accumulator registers = (quad % 4) / 2.
  const int vt_off = ((ld_row >> 2) * 2 + (ld_row & 1)) * 16 + ((ld_row & 3) >> 1) * 8;

  auto store_tile = [&](int stage) {
    unsigned char* ks = smem + stage * kStageBytes;
    unsigned char* vs = ks + kKBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<u32x4*>(ks + (ld_row + 16 * i) * (kKStride * 2) + ld_chunk * 16) = kreg[i];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // dword j of each row holds head-dim values 2j (low half) and 2j+1 (high half)
      u32x2 even, odd;
      even[0] = __builtin_amdgcn_perm(vreg[1][j], vreg[0][j], 0x05040100u);
      even[1] = __builtin_amdgcn_perm(vreg[3][j], vreg[2][j], 0x05040100u);
      odd[0] = __builtin_amdgcn_perm(vreg[1][j], vreg[0][j], 0x07060302u);
      odd[1] = __builtin_amdgcn_perm(vreg[3][j], vreg[2][j], 0x07060302u);
      const int d = ld_chunk * 8 + 2 * j;
      *reinterpret_cast<u32x2*>(vs + d * (kVStride * 2) + vt_off) = even;
      *reinterpret_cast<u32x2*>(vs + (d + 1) * (kVStride * 2) + vt_off) = odd;
    }
  };

  // ---- accumulators -----------------------------------------------------------------------------
  f32x16 o_acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) o_acc[i][j] = 0.f;
  float m_run = -INFINITY;   // running max of the raw (unscaled) scores of this lane's Q row
  float l_run = 0.f;         // this lane's share of the running sum (the other 32 keys: lane ^ 32)

  const int k_rd = ln * (kKStride * 2) + hf * 16;   // + mb*32*272 + ks*32
  const int v_rd = ln * (kVStride * 2) + hf * 16;   // + db*32*144 + kstep*32
  const int causal_shift = p.Sc - p.Sq;

  if (ntiles > 0) {
    load_tile(0);
    store_tile(0);
  }

  for (int t = 0; t < ntiles; ++t) {
    const int stage = t & 1;
    if (t + 1 < ntiles) load_tile(t + 1);
    __syncthreads();
    const unsigned char* ks = smem + stage * kStageBytes;
    const unsigned char* vs = ks + kKBytes;

    // ---- S^T tile: 64 keys x 32 q rows per wave ---------------------------------------------------
    f32x16 s[2];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int j = 0; j < 16; ++j) s[mb][j] = 0.f;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(ks + k_rd + mb * (32 * kKStride * 2) + kk * 32);
        s[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[kk], s[mb], 0, 0, 0);
      }
    }

    // ---- mask: keys past the chunk end, and the causal diagonal ---------------------------------
    const int kv0 = t * kBN;
    bool need_mask = kv0 + kBN > p.Sc;
    if (CAUSAL) need_mask = need_mask || (kv0 + kBN - 1 > q0 + causal_shift);
    if (need_mask) {
      int lim = p.Sc - 1;                                   // last visible key of this lane's row
      if (CAUSAL) { const int c = my_q + causal_shift; lim = c < lim ? c : lim; }
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int key = kv0 + mb * 32 + (j >> 2) * 8 + hf * 4 + (j & 3);
          if (key > lim) s[mb][j] = -INFINITY;
        }
    }

    // ---- online softmax (per lane = per Q row) ----------------------------------------------------
    float mx = s[0][0];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int j = 0; j < 16; ++j) mx = fmaxf(mx, s[mb][j]);
    mx = pair_max(mx);
    const float m_new = fmaxf(m_run, mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2((m_run - m_use) * p.scale_log2);
    const float msc = m_use * p.scale_log2;
    m_run = m_new;
    float rs = 0.f;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float e = fast_exp2(__builtin_fmaf(s[mb][j], p.scale_log2, -msc));
        s[mb][j] = e;
        rs += e;
      }
    l_run = l_run * alpha + rs;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int j = 0; j < 16; ++j) o_acc[db][j] *= alpha;

    // ---- P^T as bf16 B operands: k-step (mb, j2) takes accumulator registers 8 j2 .. 8 j2 + 7 ---
    bf16x8 pf[4];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int j2 = 0; j2 < 2; ++j2) {
        u32x4 w;
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = pack_bf16(s[mb][8 * j2 + 2 * e], s[mb][8 * j2 + 2 * e + 1]);
        pf[mb * 2 + j2] = __builtin_bit_cast(bf16x8, w);
      }

    // ---- O^T += V^T P^T ----------------------------------------------------------------------------
#pragma unroll
    for (int kstep = 0; kstep < 4; ++kstep) {
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const bf16x8 vf = *reinterpret_cast<const bf16x8*>(vs + v_rd + db * (32 * kVStride * 2) + kstep * 32);
        o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kstep], o_acc[db], 0, 0, 0);
      }
    }

    if (t + 1 < ntiles) store_tile(stage ^ 1);
  }

  // ---- epilogue -----------------------------------------------------------------------------------
  const float l_tot = pair_sum(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (hf == 0 && my_q < p.Sq) {
    const float lse = l_tot > 0.f ? m_run * p.scale + fast_log2(l_tot) * kLn2 : -INFINITY;
    p.lse[((int64_t)b * p.Hq + hq) * p.Sq + my_q] = lse;
  }

  __syncthreads();   // every wave is done with the K/V tiles: reuse LDS to transpose O
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

int attn_fwd_bf16(const void* q, const void* k, const void* v, void* out, float* lse,
                  int B, int Sq, int Sc, int Hq, int Hkv,
                  const int64_t* st, float scale, int mask, hipStream_t stream) {
  FwdParams p;
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.out = static_cast<uint16_t*>(out);
  p.lse = lse;
  p.B = B; p.Sq = Sq; p.Sc = Sc; p.Hq = Hq; p.Hkv = Hkv; p.group = Hq / Hkv;
  p.q_sb = st[0]; p.q_ss = st[1]; p.q_sh = st[2];
  p.k_sb = st[3]; p.k_ss = st[4]; p.k_sh = st[5];
  p.v_sb = st[6]; p.v_ss = st[7]; p.v_sh = st[8];
  p.o_sb = st[9]; p.o_ss = st[10]; p.o_sh = st[11];
  p.scale = scale;
  p.scale_log2 = scale * kLog2e;
  p.nq_tiles = (Sq + kBM - 1) / kBM;
  p.total = B * Hq * p.nq_tiles;
  p.per_xcd = (p.total + 7) / 8;
  const dim3 grid(p.per_xcd * 8), block(kThreads);
  if (mask == MHIP_MASK_CAUSAL)
    hipLaunchKernelGGL(attn_fwd_bf16_d128<true>, grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL(attn_fwd_bf16_d128<false>, grid, block, 0, stream, p);
  return launch_status();
}

}  // namespace mhip
