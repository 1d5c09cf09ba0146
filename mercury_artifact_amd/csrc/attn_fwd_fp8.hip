// Block forward on e4m3 (OCP float8) Q/K/V for gfx950: out = softmax(scale * q k^T) v in bf16 and
// lse in fp32, with x ~ descale_x * x_q per tensor.  Both contractions run on the 64-deep fp8 MFMA
// (v_mfma_f32_32x32x64_f8f6f4, twice the rate of the bf16 one), fp32 softmax.  Not in the reference; same
// call boundary as the bf16 kernel (utils/flash_attn_dsl.py:159-176) with three extra descale arguments.
//
// Same decomposition as the bf16 kernel: 8 wavefronts x 32 Q rows per workgroup, S^T = K Q^T keeps one Q
// row per lane, P^T feeds the second MFMA from the accumulator registers, K and V tiles are copied
// global -> LDS without registers in between, four stages deep.  Differences:
//   * a main-loop tile is 128 keys (as many bytes as the 64-key bf16 tile), rows of 128 bytes whose eight
//     16-byte chunks are XOR-swizzled;
//   * an MFMA takes 32 bytes per lane and operand: for S^T two 16-byte LDS reads of one K row, for O^T four
//     ds_read_b64_tr_b8 of the row-major V tile (8 keys of one head-dim column each);
//   * the K rows of a 32-key block are assigned to the MFMA rows through a permutation chosen so that a
//     lane's 16 accumulator registers hold 16 CONSECUTIVE keys (16 hf + i): the transposing reads, which
//     deliver 8 consecutive keys, then produce V^T in exactly the key order of the P registers;
//   * the descales fold into the softmax scale (q, k) and the final normalisation (v);
//   * P is multiplied by 2^4 before it is rounded to e4m3 (and the result divided by 2^4), so that small
//     probabilities keep their relative precision; the reference score of a row is its first tile's maximum
//     and moves only when the sum of a group of 16 values of 2^4 P reaches the e4m3 maximum of 448 (the sums
//     are watched, not the maxima: the common path has no maximum, no cross-lane exchange, no rescale of O).
#include "mhip_common.hpp"

namespace mhip {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(int)))) int i32x8;
typedef __attribute__((__vector_size__(2 * sizeof(int)))) int i32x2;

constexpr int kD = 128;
constexpr int kWaves = 8;
constexpr int kBM = kWaves * 32;
constexpr int kBN = 128;              // keys per tile
constexpr int kTileBytes = kBN * kD;  // 16384: one K or V tile in LDS, 128 rows of 128 bytes
constexpr int kStages = 4;
constexpr int kVBase = kStages * kTileBytes;
constexpr int kOStride = kD + 8;
constexpr float kPShift = 4.f;        // P is stored as 2^4 P in e4m3
constexpr float kTrigger = 448.f;     // the e4m3 maximum: a group of 16 exponentials has to sum to less
constexpr int kNoColumn = 0x7fff0000;  // vector offset that is out of every descriptor's range (spans stay below 2^30
                                       // when it is used, and so does the scalar tile offset added to it)

struct Fp8Params {
  const uint8_t* q; const uint8_t* k; const uint8_t* v;
  uint16_t* out; float* lse;
  int B, Sq, Sc, Hq, Hkv, group;
  int D;             // head dimension of the tensors, a multiple of 16 up to kD; columns D .. kD-1 are zeros on chip
  int64_t q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, v_sb, v_ss, v_sh, o_sb, o_ss, o_sh;
  float scale;           // softmax scale
  const float* q_descale; const float* k_descale; const float* v_descale;   // device scalars, NULL = 1
  int nq_tiles, total, per_xcd, heads_per_xcd;
};

// Chunk c (16 bytes) of row r of a tile lives at chunk position c ^ swz8(r).  Row pairs share a 256-byte
// bank line, so the position inside the line is (r & 1, c ^ swz8(r)): the 32 rows of one 16-byte operand
// read and the 16 rows x 2 chunks of one transposing read both cover the 16 positions exactly twice.
__device__ __forceinline__ constexpr int swz8(int row) { return (((row >> 1) & 3) << 1) | ((row >> 3) & 1); }

template <bool CAUSAL>
__global__ __launch_bounds__(kWaves * 64, 2) void attn_fwd_fp8_d128(const Fp8Params p) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * kStages * kTileBytes];

  // The per-tensor descales are read from device memory here (one scalar load each), so a step whose operands are
  // re-quantised every time needs no device-to-host copy and a captured graph sees the values of the replay.
  const float qd = p.q_descale ? *p.q_descale : 1.f;
  const float kd = p.k_descale ? *p.k_descale : 1.f;
  const float out_mul = p.v_descale ? *p.v_descale : 1.f;
  const float scale_eff = p.scale * qd * kd;      // natural-log scale of the integer-like dot
  const float scale_log2 = scale_eff * kLog2e;

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

  int kv_end = p.Sc;
  if (CAUSAL) {
    const int lim = q0 + kBM + (p.Sc - p.Sq);
    kv_end = lim < kv_end ? lim : kv_end;
    if (kv_end < 0) kv_end = 0;
  }
  const int ntiles = (kv_end + kBN - 1) / kBN;

  // ---- Q fragment: B operand of S^T, lane (ln, hf) holds bytes [64 ks + 32 hf, +32) of its row ------------
  const int my_q = q0 + wave * 32 + ln;
  i32x8 qf[2];    // loaded after the first tile copies are under way, so that one wait covers both latencies

  // ---- global -> LDS copies: wavefront w copies rows 16w .. 16w+15 of every K and V tile with two
  // instructions of 1 KB; lane l of instruction u lands at row 16w + 8u + l/8, chunk position l%8, and
  // fetches the chunk that lives there.  Rows past the end of the chunk arrive as zeros. ---------------------
  // Chunks past the head dimension (D < 128) carry an offset that is out of range for every tile and arrive as
  // zeros too: a tile in LDS always has 128 columns, at no cost in memory traffic.
  const u32x4 krs = rsrc_words(p.k + b * p.k_sb + hk * p.k_sh, (uint32_t)((int64_t)(p.Sc - 1) * p.k_ss + p.D));
  const u32x4 vrs = rsrc_words(p.v + b * p.v_sb + hk * p.v_sh, (uint32_t)((int64_t)(p.Sc - 1) * p.v_ss + p.D));
  int kvoff[2], vvoff[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int row = 16 * wave + 8 * u + (lane >> 3);
    const int chunk = (lane & 7) ^ swz8(row);
    const bool real = chunk * 16 < p.D;
    kvoff[u] = real ? (int)(row * p.k_ss) + chunk * 16 : kNoColumn;
    vvoff[u] = real ? (int)(row * p.v_ss) + chunk * 16 : kNoColumn;
  }
  const int k_tile_bytes = (int)(kBN * p.k_ss);
  const int v_tile_bytes = (int)(kBN * p.v_ss);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem + wave * 2048;
  auto copy_tile = [&](int t, int stage) {
#pragma unroll
    for (int u = 0; u < 2; ++u) copy16_to_lds(krs, lds_base + stage * kTileBytes + u * 1024, kvoff[u], t * k_tile_bytes);
#pragma unroll
    for (int u = 0; u < 2; ++u)
      copy16_to_lds(vrs, lds_base + kVBase + stage * kTileBytes + u * 1024, vvoff[u], t * v_tile_bytes);
  };

  // K operand of S^T: MFMA row m of block mb is key 32 mb + pi(m), pi(8 g + 4 h + e) = 16 h + 4 g + e, so
  // that accumulator register i of lane half hf is key 32 mb + 16 hf + i.  The lane reads chunks
  // 4 ks + 2 hf and 4 ks + 2 hf + 1 of that row.
  const int pi = 16 * ((ln >> 2) & 1) + 4 * (ln >> 3) + (ln & 3);
  int k_rd[2][2];                                     // [ks][second 16 bytes]  + mb * 4096
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int u = 0; u < 2; ++u) k_rd[ks][u] = pi * 128 + (((4 * ks + 2 * hf + u) ^ swz8(pi)) << 4);
  // V^T operand of O^T for head-dim block db and k-step ks2 (keys 64 ks2 .. +63): bytes 8 n .. 8 n + 7 of
  // the lane's 32 are keys 64 ks2 + 32 (n / 2) + 16 hf + 8 (n % 2) + 0..7, the keys of its P registers.
  // One ds_read_b64_tr_b8 per n: within 16 lanes, lane s supplies the address of row (first key) + s/2,
  // head-dim bytes 8 (s%2) .. +7 of the 16-column strip, and receives column s.
  int v_rd[4][2];                                     // [db][n % 2]  + ks2 * 8192 + (n / 2) * 4096
  {
    const int s16 = lane & 15, strip = (lane >> 4) & 1;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int o = 0; o < 2; ++o) {
        const int row = 16 * hf + 8 * o + (s16 >> 1);
        v_rd[db][o] = row * 128 + (((2 * db + strip) ^ swz8(row)) << 4) + (s16 & 1) * 8;
      }
  }
  typedef __attribute__((address_space(3))) i32x2* lds_i32x2;
  auto read_k = [&](const unsigned char* ks_, int mb, int ks) -> i32x8 {
    const u32x4 lo = *reinterpret_cast<const u32x4*>(ks_ + k_rd[ks][0] + mb * 4096);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(ks_ + k_rd[ks][1] + mb * 4096);
    i32x8 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) { r[e] = (int)lo[e]; r[4 + e] = (int)hi[e]; }
    return r;
  };
  auto read_v = [&](const unsigned char* vs_, int db, int ks2) -> i32x8 {
    i32x8 r;
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const i32x2 t = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
          (lds_i32x2)(vs_ + v_rd[db][n & 1] + ks2 * 8192 + (n >> 1) * 4096));
      r[2 * n] = t[0]; r[2 * n + 1] = t[1];
    }
    return r;
  };
  const int causal_shift = p.Sc - p.Sq;

  f32x16 o_acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) o_acc[i][j] = 0.f;
  // m_ref: the raw score the exponentials of this lane's Q row are taken relative to.  It is set to the first
  // tile's row maximum and moves only when a later tile would overflow e4m3: what is watched is the sum of each
  // group of 16 exponentials (one compare per tile), not the maxima.  A group sum below 448 means every 2^4 P in
  // it is below the e4m3 maximum; P = 1 for all 16 gives 256.  When a sum reaches 448 the reference moves up to
  // the row maximum seen so far (O and the running sum are rescaled) and the tile's exponentials are redone, after
  // which every 2^4 P is at most 16.
  float m_ref = 0.f, msc = -kPShift, l_run = 0.f;      // l_run sums 2^4 P (this lane's half of the keys)
  float rs_sum = 0.f;
  i32x8 pf[2] = {};          // P^T operands; pf[ks2]: dwords 0-3 = keys of block 2 ks2, dwords 4-7 = block 2 ks2 + 1
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  f32x16 s[4];               // S^T tile: 128 keys x 32 q rows per wave
  auto set_reference = [&](bool first) {
    float mx = s[0][0];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int j = 0; j < 16; ++j) mx = fmaxf(mx, s[mb][j]);
    mx = pair_max(mx);
    const bool move = first ? (mx != -INFINITY) : (mx > m_ref);      // false for NaN
    if (!first) {
      const float alpha = move ? fast_exp2((m_ref - mx) * scale_log2) : 1.f;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int j = 0; j < 16; ++j) o_acc[db][j] *= alpha;
    }
    m_ref = move ? mx : m_ref;
    msc = m_ref * scale_log2 - kPShift;            // exponent of 2^4 P
  };
  // 2^4 P of the tile into the P^T operands; returns whether one of the four group sums reached the trigger (or is
  // inf / NaN) and leaves their total in rs_sum.  s stays intact, so that the pass can be repeated against a new
  // reference.
  auto exponentials = [&]() -> bool {
    bool big = false;
    rs_sum = 0.f;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      float e[16];
      float r = 0.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        e[j] = fast_exp2(__builtin_fmaf(s[mb][j], scale_log2, -msc));
        r += e[j];
      }
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        // the first conversion writes the low half and the second the high half of the operand register, so
        // what it held before (the P of the previous tile) needs no clearing
        int packed = pf[mb >> 1][(mb & 1) * 4 + w];
        packed = __builtin_amdgcn_cvt_pk_fp8_f32(e[4 * w], e[4 * w + 1], packed, false);
        packed = __builtin_amdgcn_cvt_pk_fp8_f32(e[4 * w + 2], e[4 * w + 3], packed, true);
        pf[mb >> 1][(mb & 1) * 4 + w] = packed;
      }
      big = big || !(r < kTrigger);
      rs_sum += r;
    }
    return big;
  };

  // Tile t lives in stage t % 4 of the K and the V ring.  An iteration starts by waiting for this
  // wavefront's copies of tile t (those of tiles t+1 and t+2 stay in flight) and a barrier: after it tile t
  // is complete for every wavefront and nobody reads tile t-1 any more, whose stages then receive tile t+3.
  // Tiles past the end are copied as zeros so that the number of copies in flight stays the same.
  if (ntiles > 0) {
    copy_tile(0, 0);
    copy_tile(1, 1);
    copy_tile(2, 2);
  }
  {
    const int row = my_q < p.Sq ? my_q : p.Sq - 1;
    const uint8_t* qp = p.q + b * p.q_sb + (int64_t)row * p.q_ss + hq * p.q_sh + hf * 32;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const u32x4 none = {0u, 0u, 0u, 0u};                        // columns past the head dimension
      const int col = ks * 64 + hf * 32;
      const u32x4 lo = col < p.D ? *reinterpret_cast<const u32x4*>(qp + ks * 64) : none;
      const u32x4 hi = col + 16 < p.D ? *reinterpret_cast<const u32x4*>(qp + ks * 64 + 16) : none;
#pragma unroll
      for (int e = 0; e < 4; ++e) { qf[ks][e] = (int)lo[e]; qf[ks][4 + e] = (int)hi[e]; }
    }
    // pin the loads here: the copies are invisible to the compiler's wait counting
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) asm volatile("" : "+v"(qf[ks]));
  }
  for (int t = 0; t < ntiles; ++t) {
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");      // two tiles of four copies each
    __builtin_amdgcn_s_barrier();
    copy_tile(t + 3, (t + 3) & 3);
    const unsigned char* ks_ = smem + (t & 3) * kTileBytes;
    const unsigned char* vs_ = smem + kVBase + (t & 3) * kTileBytes;

    // ---- S^T tile ---------------------------------------------------------------------------------------
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) {
        const i32x8 kf = read_k(ks_, mb, ks);
        s[mb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf, qf[ks], ks == 0 ? zero : s[mb], 0, 0, 0, 0, 0, 0);
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
          const int key = kv0 + mb * 32 + hf * 16 + j;
          if (key > lim) s[mb][j] = -INFINITY;
        }
    }

    // ---- softmax against a reference that moves only when it has to -----------------------------------------
    if (t == 0) set_reference(true);
    if (__builtin_amdgcn_ballot_w64(exponentials()) != 0) {
      set_reference(false);
      exponentials();
    }
    l_run += rs_sum;

    // ---- O^T += V^T P^T -----------------------------------------------------------------------------------
#pragma unroll
    for (int ks2 = 0; ks2 < 2; ++ks2) {
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const i32x8 vf = read_v(vs_, db, ks2);
        o_acc[db] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf, pf[ks2], o_acc[db], 0, 0, 0, 0, 0, 0);
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the zero-filled copies of tiles past the end

  // ---- epilogue ---------------------------------------------------------------------------------------------
  const float l_tot = pair_sum(l_run);
  const float inv = l_tot > 0.f ? out_mul / l_tot : 0.f;           // the two factors 2^4 cancel
  if (hf == 0 && my_q < p.Sq) {
    const float lse = l_tot > 0.f ? m_ref * scale_eff + (fast_log2(l_tot) - kPShift) * kLn2 : -INFINITY;
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
      if (row < p.Sq && chunk * 8 < p.D) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(os + r * (kOStride * 2) + chunk * 16);
        *reinterpret_cast<u32x4*>(op + (int64_t)row * p.o_ss) = w;
      }
    }
  }
}

}  // namespace

int attn_fwd_fp8(const void* q, const void* k, const void* v, void* out, float* lse,
                 int B, int Sq, int Sc, int Hq, int Hkv, int D, const int64_t* st, float scale, int mask,
                 const float* q_descale, const float* k_descale, const float* v_descale, hipStream_t stream) {
  Fp8Params p;
  p.q = static_cast<const uint8_t*>(q); p.k = static_cast<const uint8_t*>(k); p.v = static_cast<const uint8_t*>(v);
  p.out = static_cast<uint16_t*>(out); p.lse = lse;
  p.B = B; p.Sq = Sq; p.Sc = Sc; p.Hq = Hq; p.Hkv = Hkv; p.group = Hq / Hkv;
  p.D = D;
  p.q_sb = st[0]; p.q_ss = st[1]; p.q_sh = st[2];
  p.k_sb = st[3]; p.k_ss = st[4]; p.k_sh = st[5];
  p.v_sb = st[6]; p.v_ss = st[7]; p.v_sh = st[8];
  p.o_sb = st[9]; p.o_ss = st[10]; p.o_sh = st[11];
  p.scale = scale;
  p.q_descale = q_descale; p.k_descale = k_descale; p.v_descale = v_descale;
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
