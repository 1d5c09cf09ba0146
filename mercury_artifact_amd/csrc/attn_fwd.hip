// Block forward of the ring-attention step for gfx950: one Q shard against one KV chunk,
// out = softmax(scale * q k^T) v and lse = logsumexp(scale * q k^T), bf16 in, fp32 accumulate.
//
// Replaces the flash-attn call at utils/flash_attn_dsl.py:159-176 of the reference.
//
// Work decomposition
//   workgroup  = 256 Q rows of one (batch, q-head): 8 wavefronts x 32 rows, one workgroup per CU,
//                two wavefronts per SIMD
//   main loop  = 64-key tiles of the chunk.  K and V tiles go from global memory straight into LDS
//                (buffer_load ... lds, no registers in between), row-major with the 16-byte chunks of
//                a row XOR-swizzled, four stages each; every wavefront copies 8 rows of each tile
//   S^T = K Q^T  : v_mfma_f32_32x32x16_bf16 with A = K rows (LDS), B = Q (registers, loaded once).
//                  The accumulator layout puts one Q row in each lane (lane % 32) and 32 of the
//                  64 keys of the tile in that lane's registers, so the softmax is lane-local.
//   O^T = V^T P^T: the same lane that produced P^T[key][q] feeds it back as the B operand; the
//                  key order inside one MFMA k-step is whatever the accumulator registers hold, and
//                  the V^T operand is gathered in exactly that order from the row-major V tile by
//                  ds_read_b64_tr_b16 (four keys of one head-dim column per lane), so P never moves.
//   ping-pong    : every tile is split into a matrix phase (S^T of the next tile + O^T of this one,
//                  32 MFMAs) and a vector phase (softmax of the next tile, tile copies).  Wavefronts
//                  0-3 and 4-7 run half a tile apart, separated by workgroup barriers, so on every
//                  SIMD one wavefront feeds the matrix pipe while the other does exponentials.
//   softmax      : the reference score of a row is fixed by the first tile's row maximum and moves only
//                  when a later tile would overflow: the row SUMS are watched (one compare per tile),
//                  not the maxima, so the common path has no maximum, no cross-lane exchange and no
//                  rescale of O; two of a tile's sixteen pairs of exponentials ride behind the last
//                  MFMAs of the matrix phase (the vector phase was the longer of the two).
#include "mhip_common.hpp"

namespace mhip {
namespace {

constexpr int kD = 128;            // head dimension
constexpr int kWaves = 8;
constexpr int kBM = kWaves * 32;   // Q rows per workgroup
constexpr int kBN = 64;            // keys per main-loop tile
constexpr int kTileBytes = kBN * kD * 2;   // 16384: one K or V tile in LDS, 64 rows of 256 bytes
constexpr int kStages = 4;                 // K(t+1) .. K(t+4) and V(t) .. V(t+3) live while tile t is processed
constexpr int kVBase = kStages * kTileBytes;
constexpr int kOStride = kD + 8;   // epilogue staging of O, bf16 elements per row
constexpr int kNoColumn = 0x7fff0000;  // vector offset that is out of every descriptor's range (spans stay below 2^31,
                                       // and so does the scalar tile offset added to it: no 32-bit wrap)
constexpr int kFragDepth = 4;      // LDS operand reads in flight ahead of the MFMAs (6 and 8 measure the same)
constexpr int kEarlyPairs = 2;     // exponential pairs of a tile computed inside the matrix phase (4 .. 8: 1-3 % slower)
constexpr int kEarlyStep = 2;      // matrix-phase slots between them

struct FwdParams {
  const uint16_t* q; const uint16_t* k; const uint16_t* v;
  uint16_t* out; float* lse;
  int B, Sq, Sc, Hq, Hkv, group;
  int D;             // head dimension of the tensors, a multiple of 8 up to kD; columns D .. kD-1 are zeros on chip
  int64_t q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, v_sb, v_ss, v_sh, o_sb, o_ss, o_sh;
  float scale, scale_log2;
  int nq_tiles;      // ceil(Sq / rows per workgroup)
  int total;         // B * Hq * nq_tiles
  int per_xcd;       // ceil(total / 8)
  int heads_per_xcd; // (batch, head) pairs per XCD when they divide evenly, else 0
};

// KK = k-steps of 16 head-dim values in S^T: 8 computes on all 128 on-chip columns; 4 is the instantiation for head
// dimensions up to 64, which leaves out the MFMAs that would only see the zero columns (half of both products).
template <bool CAUSAL, int KK = 8>
__global__ __launch_bounds__(kWaves * 64, 2) void attn_fwd_bf16_d128(const FwdParams p) {
  static_assert(KK == 8 || KK == 4, "128 or 64 on-chip head-dim columns");
  constexpr int DB = KK / 2;        // blocks of 32 head-dim values in O^T
  constexpr int kSlotsS = 2 * KK;   // matrix-phase slots of S^T (two 32-key blocks per k-step)
  constexpr int kSlotsO = 4 * DB;   // and of O^T (four k-steps of 16 keys per block)
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * kStages * kTileBytes];

  // Workgroup i runs on XCD i % 8.  Give every XCD a contiguous range of the (batch, head, q-tile)
  // order so that the workgroups sharing one K/V head also share one L2.
  // Under the causal mask a Q tile's work grows with its index, so there the order is longest tiles
  // first across all heads (of the XCD when the heads divide evenly over the XCDs, of the launch
  // otherwise): the short tiles fill the tail.
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
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: role branches stay uniform
  const int lane = tid & 63;
  const int ln = lane & 31;
  const int hf = lane >> 5;
  const bool group_b = wave >= 4;                 // second ping-pong group

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
  bf16x8 qf[KK];  // loaded in the prologue, after the first tile copies are under way

  // ---- global -> LDS copies of the K and V tiles ---------------------------------------------------
  // A tile is 64 rows of 256 bytes.  Chunk c (16 bytes) of row r lives at chunk position c ^ swz(r):
  // the 32 rows a b128 operand read touches then spread over all banks, and so do the 8 rows x 4 chunks
  // of a transposing read.  Wavefront w copies rows 8w .. 8w+7 of every tile with two instructions of
  // 1 KB; lane l of instruction u lands at row 8w + 4u + l/16, position l%16 (the hardware places the
  // lanes back to back) and therefore fetches chunk (l%16) ^ swz(row).  Rows past the end of the chunk
  // are out of the descriptor's range and arrive as zeros, and so do the chunks past the head dimension
  // when it is below 128: their lanes carry an offset that is out of range for every tile, so a tile in
  // LDS always has 128 columns, the upper ones zero, at no cost in memory traffic.
  auto swz = [](int row) { return lds_row_swizzle(row); };
  const u32x4 krs = rsrc_words(p.k + b * p.k_sb + hk * p.k_sh, (uint32_t)(((int64_t)(p.Sc - 1) * p.k_ss + p.D) * 2));
  const u32x4 vrs = rsrc_words(p.v + b * p.v_sb + hk * p.v_sh, (uint32_t)(((int64_t)(p.Sc - 1) * p.v_ss + p.D) * 2));
  int kvoff[2], vvoff[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int row = 8 * wave + 4 * u + (lane >> 4);
    const int chunk = (lane & 15) ^ swz(row);
    const bool real = chunk * 8 < p.D;
    kvoff[u] = real ? (int)(row * p.k_ss * 2) + chunk * 16 : kNoColumn;
    vvoff[u] = real ? (int)(row * p.v_ss * 2) + chunk * 16 : kNoColumn;
  }
  const int k_tile_bytes = (int)(kBN * p.k_ss * 2);
  const int v_tile_bytes = (int)(kBN * p.v_ss * 2);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem + wave * 2048;
  auto copy_k = [&](int t, int stage) {
#pragma unroll
    for (int u = 0; u < 2; ++u) copy16_to_lds(krs, lds_base + stage * kTileBytes + u * 1024, kvoff[u], t * k_tile_bytes);
  };
  auto copy_v = [&](int t, int stage) {
#pragma unroll
    for (int u = 0; u < 2; ++u)
      copy16_to_lds(vrs, lds_base + kVBase + stage * kTileBytes + u * 1024, vvoff[u], t * v_tile_bytes);
  };

  // K operand of S^T (A, 32 keys x 16 head-dim values): lane (ln, hf) reads chunk 2 kk + hf of row
  // 32 mb + ln.
  int k_rd[KK];                                       // + mb * 8192
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) k_rd[kk] = ln * 256 + (((2 * kk + hf) ^ swz(ln)) << 4);
  // V^T operand of O^T (A, 32 head-dim values x 16 keys) for head-dim block db and k-step (mb, j2): the
  // lane's 8 keys are rows R + {0..3} and R + 8 + {0..3}, R = 32 mb + 16 j2 + 4 hf -- the keys its P
  // registers hold.  One ds_read_b64_tr_b16 per group of 4 rows: within 16 lanes, lane s supplies the
  // address of row R + s/4, head-dim values 4 (s%4) .. +3 of the 16-column strip, and receives column s.
  int v_rd[DB][2];                                    // [db][second four rows]  + mb * 8192 + j2 * 4096
  {
    const int s16 = lane & 15, strip = (lane >> 4) & 1;
    const int cl = 2 * strip + ((s16 & 3) >> 1);
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int row = 8 * h + 4 * hf + (s16 >> 2);
        v_rd[db][h] = row * 256 + (((4 * db + cl) ^ swz(row)) << 4) + (s16 & 1) * 8;
      }
  }
  typedef __attribute__((address_space(3))) bf16x4* lds_bf16x4;
  auto read_k = [&](const unsigned char* ks, int mb, int kk) -> bf16x8 {
    return *reinterpret_cast<const bf16x8*>(ks + k_rd[kk] + mb * 8192);
  };
  auto read_v = [&](const unsigned char* vs, int db, int kstep) -> bf16x8 {
    const unsigned char* base = vs + (kstep >> 1) * 8192 + (kstep & 1) * 4096;
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4)(base + v_rd[db][0]));
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4)(base + v_rd[db][1]));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  const int causal_shift = p.Sc - p.Sq;

  // ---- accumulators -----------------------------------------------------------------------------
  f32x16 o_acc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) o_acc[i][j] = 0.f;
  // m_ref: the raw (unscaled) score the exponentials of this lane's Q row are taken relative to.  It is
  // fixed by the first tile's row maximum and moves only when a later tile would overflow: the row sums are
  // watched, not the maxima, so the common path has no maximum, no cross-lane exchange and no rescale of O.
  float m_ref = 0.f;
  float nmsc = 0.f;          // -m_ref * scale * log2(e)
  float l_run = 0.f;         // this lane's share of the running sum (the other 32 keys: lane ^ 32)
  constexpr float kTrigger = 1048576.f;   // a lane's 32 exponentials of one tile sum to less than this, or
  constexpr float kSlack = 14.f;          // rows whose maximum exceeds the reference by 2^kSlack move it
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  f32x16 s[2];               // S^T tile: 64 keys x 32 q rows per wave
  u32x4 pw[4];               // P^T of the current tile as packed bf16 B operands, one per k-step

  auto qk = [&](int stage) {
    const unsigned char* ks = smem + stage * kTileBytes;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        const bf16x8 kf = read_k(ks, mb, kk);
        s[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[kk], kk == 0 ? zero : s[mb], 0, 0, 0);
      }
    }
  };

  auto pv = [&](int stage) {
    const unsigned char* vs = smem + kVBase + stage * kTileBytes;
#pragma unroll
    for (int kstep = 0; kstep < 4; ++kstep) {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const bf16x8 vf = read_v(vs, db, kstep);
        o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, __builtin_bit_cast(bf16x8, pw[kstep]), o_acc[db], 0, 0, 0);
      }
    }
  };

  // keys past the chunk end and the causal diagonal -> -inf
  auto sm_mask = [&](int t) {
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
  };
  // Exponentials of the tile in 16 pairs: pair idx covers accumulator registers 2 idx, 2 idx + 1 (counted over
  // both 32-key blocks) and gives one dword of the packed P^T operand of k-step idx / 4.  s stays intact.
  // The first kEarlyPairs pairs are computed inside the matrix phase, between the O^T MFMAs: measured with
  // cycle counters the vector phase is the longer of the two (1314 against 1265 ticks per 64-key tile), and
  // two pairs moved over make the step 3 % faster (four and more slow the matrix phase down by as much as
  // they shorten the other).  A pair may overwrite the P^T operand of k-step ks only after the last MFMA of
  // that k-step has been issued.
  float rs = 0.f;
  auto sm_pair = [&](int idx) {
    const int mb = idx >> 3, r = (idx & 7) * 2;
    float x0 = fast_exp2(__builtin_fmaf(s[mb][r], p.scale_log2, nmsc));
    float x1 = fast_exp2(__builtin_fmaf(s[mb][r + 1], p.scale_log2, nmsc));
    if (idx == 0) rs = x0 + x1; else rs += x0 + x1;
    uint32_t w = pack_bf16(x0, x1);
    asm volatile("" : "+v"(w), "+v"(rs));          // keeps the pair where it is written
    pw[idx >> 2][idx & 3] = w;
  };
  auto sm_exps = [&]() {
#pragma unroll
    for (int idx = 0; idx < 16; ++idx) sm_pair(idx);
  };
  // Move the reference of the rows whose scores outgrew it (first tile: set it to the row maximum) and
  // rescale O and the running sum accordingly.
  auto sm_fix = [&](bool first) {
    float mx = s[0][0];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int j = 0; j < 16; ++j) mx = fmaxf(mx, s[mb][j]);
    mx = pair_max(mx);
    const float grown = (mx - m_ref) * p.scale_log2;               // NaN when mx = -inf on the first tile
    const bool move = first ? (mx != -INFINITY) : (grown > kSlack);   // false for NaN
    if (!first) {
      const float alpha = move ? fast_exp2(-grown) : 1.f;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int j = 0; j < 16; ++j) o_acc[db][j] *= alpha;
      l_run *= alpha;
    }
    m_ref = move ? mx : m_ref;
    nmsc = -m_ref * p.scale_log2;
  };
  // slot of the matrix phase after which early pair idx runs: k-step idx / 4 of the tile before is read by the
  // O^T slots kSlotsS + DB (idx / 4) .. + DB - 1, and the pairs are spread two slots apart behind that
  auto early_slot = [](int idx) {
    return idx < 4 ? kSlotsS + DB + kEarlyStep * idx : kSlotsS + 3 * DB + (idx - 4);
  };
  static_assert(kEarlyPairs <= 4 && kSlotsS + DB + kEarlyStep * (kEarlyPairs - 1) < kSlotsS + kSlotsO,
                "the early pairs have to fit behind the O^T slots of k-step 0");
  auto sm_tile = [&]() {
#pragma unroll
    for (int idx = kEarlyPairs; idx < 16; ++idx) sm_pair(idx);
    if (__builtin_amdgcn_ballot_w64(!(rs < kTrigger)) != 0) {
      sm_fix(false);
      sm_exps();
    }
    l_run += rs;
  };

  // Matrix phase of tile t: S^T(t+1) from K stage `ks_stage` and O^T += V^T(t) P^T(t) from V stage
  // `vs_stage`, kSlotsS + kSlotsO MFMAs (32 on 128 columns) fed by as many LDS reads.  The reads run kFragDepth
  // operands ahead of the MFMAs through a ring of registers, so the LDS latency is covered by the MFMAs in between.
  auto read_frag = [&](int i, const unsigned char* ks, const unsigned char* vs) -> bf16x8 {
    if (i < kSlotsS) return read_k(ks, i & 1, i >> 1);
    return read_v(vs, (i - kSlotsS) % DB, (i - kSlotsS) / DB);
  };
  // The first kFragDepth operands (all of K) are read before the barrier that opens the phase, by
  // first_frags, so the matrix pipe starts without waiting for LDS.
  bf16x8 frag[kFragDepth];
  auto first_frags = [&](int ks_stage) {
    const unsigned char* ks = smem + ks_stage * kTileBytes;
#pragma unroll
    for (int i = 0; i < kFragDepth; ++i) frag[i] = read_frag(i, ks, ks);
  };
  auto matrix_phase = [&](int t_next, int ks_stage, int vs_stage) {
    const unsigned char* ks = smem + ks_stage * kTileBytes;
    const unsigned char* vs = smem + kVBase + vs_stage * kTileBytes;
#pragma unroll
    for (int i = 0; i < kSlotsS + kSlotsO; ++i) {
      if (i < kSlotsS) {
        const int mb = i & 1, kk = i >> 1;
        s[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag[i % kFragDepth], qf[kk], kk == 0 ? zero : s[mb], 0, 0, 0);
      } else {
        const int db = (i - kSlotsS) % DB, kstep = (i - kSlotsS) / DB;
        o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag[i % kFragDepth], __builtin_bit_cast(bf16x8, pw[kstep]), o_acc[db], 0, 0, 0);
      }
      if (i + kFragDepth < kSlotsS + kSlotsO) frag[i % kFragDepth] = read_frag(i + kFragDepth, ks, vs);
      // S^T(t_next) is complete after its last slot; its softmax starts here, in the shadow of the O^T MFMAs
      if (i == kSlotsS) sm_mask(t_next);
#pragma unroll
      for (int idx = 0; idx < kEarlyPairs; ++idx)
        if (early_slot(idx) == i) sm_pair(idx);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- prologue: the first tiles into LDS, softmax of tile 0 -------------------------------------------
  // Barriers inside the loop are bare s_barrier instructions: a fence would wait for every copy in flight.
  if (ntiles > 0) {
#pragma unroll
    for (int i = 0; i < kStages; ++i) copy_k(i, i);          // tiles past the chunk arrive as zeros
#pragma unroll
    for (int i = 0; i < kStages - 1; ++i) copy_v(i, i);
  }
  {
    // The Q loads go out behind the copies, so that one wait covers both latencies.  The fragment is
    // pinned here: otherwise its first use sits inside the main loop and so does the wait for it.
    const int row = my_q < p.Sq ? my_q : p.Sq - 1;
    const uint16_t* qp = p.q + b * p.q_sb + (int64_t)row * p.q_ss + hq * p.q_sh + hf * 8;
#pragma unroll
    for (int ks = 0; ks < KK; ++ks) {
      if (ks * 16 + hf * 8 < p.D) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + ks * 16);
      else qf[ks] = bf16x8{};                       // columns past the head dimension
    }
#pragma unroll
    for (int ks = 0; ks < KK; ++ks) asm volatile("" : "+v"(qf[ks]));
  }
  if (ntiles > 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    qk(0);
    sm_mask(0);
    sm_fix(true);
    sm_exps();
    l_run = rs;
    if (ntiles > 1) first_frags(1);
  }
  // Phase p of the main loop: group A (waves 0-3) runs the matrix phase of tile p/2 on even p and its
  // vector phase on odd p; group B does the same one phase later.  K(t) and V(t) live in stage t % 4 of
  // their rings.  In the vector phase of tile t every wavefront starts its share of the copies of K(t+4)
  // (over K(t), last read in the matrix phase of tile t-1) and V(t+3) (over V(t-1)), and before the
  // barrier that ends the phase waits for the copies it started one tile earlier: those are then visible
  // to every wavefront two barriers later, in time for first_frags of K(t+3) and the matrix phase of V(t+2).
  if (group_b) __builtin_amdgcn_s_barrier();
  for (int t = 0; t + 1 < ntiles; ++t) {
    // ---- matrix phase: S^T(t+1) = K(t+1) Q^T and O^T += V^T(t) P^T(t), first part of softmax(t+1) ------
    __builtin_amdgcn_s_setprio(2);
    matrix_phase(t + 1, (t + 1) & 3, t & 3);
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_s_barrier();
    // ---- vector phase: softmax(t+1), copies of the tiles ahead ---------------------------------------------
    asm volatile("" : "+v"(s[0]), "+v"(s[1]));      // keeps the exponentials behind the barrier
    sm_tile();
    copy_k(t + 4, t & 3);
    copy_v(t + 3, (t + 3) & 3);
    if (t + 2 < ntiles) first_frags((t + 2) & 3);             // K(t+2), for the next matrix phase
    asm volatile("s_waitcnt vmcnt(4)" ::: "memory");          // the four copies of one tile ago are done
    __builtin_amdgcn_s_barrier();
  }
  if (ntiles > 0) pv((ntiles - 1) & 3);             // last tile: nothing left to prefetch or exponentiate
  if (!group_b) __builtin_amdgcn_s_barrier();

  // ---- epilogue -----------------------------------------------------------------------------------
  const float l_tot = pair_sum(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (hf == 0 && my_q < p.Sq) {
    const float lse = l_tot > 0.f ? m_ref * p.scale + fast_log2(l_tot) * kLn2 : -INFINITY;
    p.lse[((int64_t)b * p.Hq + hq) * p.Sq + my_q] = lse;
  }

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // zero-filled copies of tiles past the end included
  __syncthreads();   // every wave is done with the K/V tiles: reuse LDS to transpose O
  unsigned char* os = smem + wave * (32 * kOStride * 2);
#pragma unroll
  for (int db = 0; db < DB; ++db)
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

int attn_fwd_bf16(const void* q, const void* k, const void* v, void* out, float* lse,
                  int B, int Sq, int Sc, int Hq, int Hkv, int D,
                  const int64_t* st, float scale, int mask, hipStream_t stream) {
  FwdParams p;
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.out = static_cast<uint16_t*>(out);
  p.lse = lse;
  p.B = B; p.Sq = Sq; p.Sc = Sc; p.Hq = Hq; p.Hkv = Hkv; p.group = Hq / Hkv;
  p.D = D;
  p.q_sb = st[0]; p.q_ss = st[1]; p.q_sh = st[2];
  p.k_sb = st[3]; p.k_ss = st[4]; p.k_sh = st[5];
  p.v_sb = st[6]; p.v_ss = st[7]; p.v_sh = st[8];
  p.o_sb = st[9]; p.o_ss = st[10]; p.o_sh = st[11];
  p.scale = scale;
  p.scale_log2 = scale * kLog2e;
  p.nq_tiles = (Sq + kBM - 1) / kBM;
  p.total = B * Hq * p.nq_tiles;
  p.per_xcd = (p.total + 7) / 8;
  p.heads_per_xcd = (B * Hq) % 8 == 0 ? (B * Hq) / 8 : 0;
  const dim3 grid(p.per_xcd * 8), block(kWaves * 64);
  const bool causal = mask == MHIP_MASK_CAUSAL;
  if (D <= 64) {        // half the on-chip columns, half the MFMAs
    if (causal) hipLaunchKernelGGL((attn_fwd_bf16_d128<true, 4>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((attn_fwd_bf16_d128<false, 4>), grid, block, 0, stream, p);
  } else {
    if (causal) hipLaunchKernelGGL((attn_fwd_bf16_d128<true, 8>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((attn_fwd_bf16_d128<false, 8>), grid, block, 0, stream, p);
  }
  return launch_status();
}

}  // namespace mhip
