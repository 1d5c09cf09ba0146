// Block backward of the ring-attention step for gfx950, recomputing P from the saved LSE.
//
// Replaces the flash-attn call at utils/attn_bwd_dsl.py:83-115 of the reference:
//     P = exp(scale * q k^T - lse),  delta = rowsum(dout * out)
//     dV = P^T dout,  dP = dout v^T,  dS = P * (dP - delta),  dQ = scale * dS k,  dK = scale * dS^T q
//
// Two kernels, launched in this order, no atomics (so every run is deterministic):
//   bwd_main<DQ=true>   one workgroup per 256 query rows of one head (eight wavefronts, two per SIMD: this pass
//                has half the accumulators of the other and fits 256 registers): Q and dout rows stay in
//                registers, K / V tiles stream through LDS; accumulates dQ.  Its prologue also works out, per
//                query row, delta = sum_d dout * out and lse2 = lse * log2(e) (with -inf, a row that saw no key,
//                turned into +inf so that P = exp2(s - lse2) = 0 there) and leaves them in the workspace
//   bwd_main<DQ=false>  one workgroup per 128 keys of one KV head: K and V rows stay in registers,
//                Q / dout tiles of the (grouped) query heads stream through LDS together with their lse2 /
//                delta from the workspace; accumulates dK, dV
// Both instances share one body.  "Stationary" rows (32 per wavefront) sit in the lane index of every
// MFMA accumulator, "streamed" rows in its registers, exactly as in the forward kernel:
//     T1[c][r] = X_str[c] . X_st[r]      (scores)          T2[c][r] = Y_str[c] . Y_st[r]      (dP)
//     acc^T[d][r] += X_str^T[d][c] dS[c][r]                (dQ or dK)
//     acc2^T[d][r] += Y_str^T[d][c] P[c][r]                (dV, DQ=false only)
// so P and dS feed the second MFMA straight from the accumulator registers.  The streamed tiles are
// copied global -> LDS without registers in between (buffer_load ... lds), row-major with swizzled
// 16-byte chunks, four stages deep; T1 / T2 read them with ds_read_b128 and the transposed operands
// of the second MFMAs are gathered from the same tiles with ds_read_b64_tr_b16, in the key order the
// accumulator registers hold.
#include "mhip_common.hpp"

#include <atomic>

namespace mhip {
namespace {

constexpr int kD = 128;
constexpr int kTile = 64;             // streamed rows per main-loop tile
constexpr int kRowsKv = 128;          // stationary key rows per workgroup of the dK / dV pass (4 wavefronts x 32)
constexpr int kRowsQ = 256;           // stationary query rows per workgroup of the dQ pass (8 wavefronts x 32)
constexpr int kTileBytes = kTile * kD * 2;             // 16384: 64 rows of 256 bytes
constexpr int kOffY = kTileBytes, kOffLse = 2 * kTileBytes, kOffDelta = kOffLse + kTile * 4;
constexpr int kStageBytes = kOffDelta + kTile * 4;     // X tile, Y tile, lse2 and delta of the streamed rows
constexpr int kStages = 4;
constexpr int kSmemBytes = kStages * kStageBytes;      // 133120
constexpr int kOStride = kD + 8;
constexpr int kNoTile = 0x7fff0000;   // scalar offset that puts every lane of a copy out of range
constexpr int kNoColumn = 0x7fff0000; // vector offset with the same effect for one lane (the sum of the two is
                                      // below 2^32: no wrap)

struct BwdParams {
  const uint16_t* q; const uint16_t* k; const uint16_t* v; const uint16_t* dout;
  const uint16_t* out; const float* lse;   // saved output and log-sum-exp of the forward
  float* lse2; float* delta;               // both (B, Hq, Sq) fp32: written by the dQ pass, read by the dK / dV pass
  float* softmax_d;                        // rowsum(dout * out) itself for the caller, or null
  uint16_t* dq; uint16_t* dk; uint16_t* dv; float* dq_acc;
  int B, Sq, Sc, Hq, Hkv, group;
  int D;            // head dimension of the tensors, a multiple of 8 up to kD; columns D .. kD-1 are zeros on chip
  int64_t q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, dk_sb, dk_ss, dk_sh, dq_sb, dq_ss, dq_sh, o_sb, o_ss, o_sh;
  float scale, scale_log2;
  int n_tiles;      // stationary tiles per (batch, head)
  int total;
  int per_xcd;
  int heads_per_xcd;   // (batch, stationary head) pairs per XCD when they divide evenly, else 0
};

template <bool DQ, bool CAUSAL>
__global__ __launch_bounds__(DQ ? 512 : 256, 1) void bwd_main(const BwdParams p) {
  // The dQ pass needs half the accumulators of the dK / dV pass and fits two wavefronts per SIMD: its workgroup
  // is eight wavefronts sharing the streamed K / V tiles.
  constexpr int kWavesWg = DQ ? 8 : 4;
  constexpr int kRowsPerWg = kWavesWg * 32;
  constexpr int kCpy = 16 / kWavesWg;           // copy instructions per wavefront for one 16 KB tile
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

  // ---- stationary operands: B operands of T1 / T2, lane (ln, hf) holds row[16 ks + 8 hf .. +7]; for dQ the
  // query is the stationary row and its lse2 / delta are per-lane scalars.  All loaded further down, behind
  // the first tile copies, so that one wait covers both latencies. ---------------------------------------
  bf16x8 xf[8], yf[8];
  float lse2_lane = 0.f, delta_lane = 0.f;

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

  const uint16_t* xbase; const uint16_t* ybase; int64_t s_ss, s_sh; uint32_t s_bytes;
  if (DQ) {
    const int hk = hs / p.group;
    xbase = p.k + b * p.k_sb + hk * p.k_sh; ybase = p.v + b * p.k_sb + hk * p.k_sh;
    s_ss = p.k_ss; s_sh = 0;
    s_bytes = (uint32_t)(((int64_t)(p.Sc - 1) * p.k_ss + p.D) * 2);
  } else {
    xbase = p.q + b * p.q_sb; ybase = p.dout + b * p.q_sb;
    s_ss = p.q_ss; s_sh = p.q_sh;
    s_bytes = (uint32_t)(((int64_t)(p.Sq - 1) * p.q_ss + (int64_t)(p.Hq - 1) * p.q_sh + p.D) * 2);
  }
  const u32x4 xrs = rsrc_words(xbase, s_bytes);
  const u32x4 yrs = rsrc_words(ybase, s_bytes);

  // tile index -> (head of the group, first streamed row)
  auto tile_head = [&](int t) { return DQ ? 0 : t / span; };
  auto tile_row0 = [&](int t) { return (first_tile + (DQ ? t : t % span)) * kTile; };

  // Wavefront w copies rows 16w .. 16w+15 of the X and the Y tile: four instructions of 1 KB each; lane l
  // of instruction u lands at row 16w + 4u + l/16, chunk position l%16, and fetches the chunk that lives
  // there.  Rows past the end of the streamed tensor arrive as zeros when the layout puts them past the
  // descriptor's range, and their P / dS are zeroed by index in any case.  lse2 and delta of the 64
  // streamed rows (DQ=false) are copied by the even / odd wavefronts (twice the same bytes: every
  // wavefront then has the same number of copies in flight, which the vmcnt waits rely on).
  int cvoff[kCpy];
#pragma unroll
  for (int u = 0; u < kCpy; ++u) {
    const int row = 4 * kCpy * wave + 4 * u + (lane >> 4);
    const int chunk = (lane & 15) ^ lds_row_swizzle(row);
    // chunks past the head dimension: an offset that is out of the descriptor's range for every tile, so they
    // arrive as zeros and a tile in LDS always has 128 columns
    cvoff[u] = chunk * 8 < p.D ? (int)(row * s_ss * 2) + (chunk << 4) : kNoColumn;
  }
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
  auto copy_tile = [&](int t, int stage) {
    const bool live = t < ntiles;
    const int hq = DQ ? 0 : hs * p.group + tile_head(live ? t : 0);
    const int c0 = tile_row0(live ? t : 0);
    const int soff = live ? (int)(((int64_t)c0 * s_ss + (int64_t)hq * s_sh) * 2) : kNoTile;
    const uint32_t dst = lds_base + stage * kStageBytes + wave * (kCpy * 1024);
#pragma unroll
    for (int u = 0; u < kCpy; ++u) copy16_to_lds(xrs, dst + u * 1024, cvoff[u], soff);
#pragma unroll
    for (int u = 0; u < kCpy; ++u) copy16_to_lds(yrs, dst + kOffY + u * 1024, cvoff[u], soff);
    if (!DQ) {
      const float* src = ((wave & 1) ? p.delta : p.lse2) + ((int64_t)b * p.Hq + hq) * p.Sq;
      copy4_to_lds(rsrc_words(src, (uint32_t)p.Sq * 4u), lds_base + stage * kStageBytes + ((wave & 1) ? kOffDelta : kOffLse),
                   lane * 4, live ? c0 * 4 : kNoTile);
    }
  };
  constexpr int kCopiesPerTile = DQ ? 2 * kCpy : 2 * kCpy + 1;
  // The same copies one instruction at a time (piece 0 .. kCopiesPerTile - 1), so that the main loop can
  // issue them between MFMAs; the scalar offsets are worked out once per tile by copy_setup.
  // Which tile comes three tiles ahead is kept as a pair of running counters (position inside the head's span,
  // head of the group) instead of a division per tile: every scalar instruction of the loop takes an issue slot of
  // the one wavefront a SIMD runs in the dK / dV pass.
  int cp_soff = 0, cp_ld_soff = 0;
  int nx_r = DQ ? 3 : (span > 0 ? 3 % span : 0), nx_h = DQ ? 0 : (span > 0 ? 3 / span : 0);
  const uint32_t ld_rows = (uint32_t)p.B * (uint32_t)p.Hq * (uint32_t)p.Sq;     // the host keeps this below 2^30
  const u32x4 ldrs = rsrc_words((wave & 1) ? p.delta : p.lse2, ld_rows * 4u);
  auto copy_setup = [&]() {
    const bool live = DQ ? nx_r < span : nx_h < heads_str;
    const uint32_t hq = DQ ? 0u : (uint32_t)(hs * p.group + (live ? nx_h : 0));
    const uint32_t c0 = (uint32_t)((first_tile + (live ? nx_r : 0)) * kTile);
    // element offsets stay below 2^31 (checked by the host), so 32-bit arithmetic is exact
    cp_soff = live ? (int)((c0 * (uint32_t)s_ss + hq * (uint32_t)s_sh) * 2u) : kNoTile;
    if (!DQ) cp_ld_soff = live ? (int)((((uint32_t)b * (uint32_t)p.Hq + hq) * (uint32_t)p.Sq + c0) * 4u) : kNoTile;
    ++nx_r;
    if (!DQ && nx_r == span) { nx_r = 0; ++nx_h; }
  };
  auto copy_piece = [&](int piece, int stage) {
    const uint32_t dst = lds_base + stage * kStageBytes + wave * (kCpy * 1024);
    if (piece < kCpy) copy16_to_lds(xrs, dst + piece * 1024, cvoff[piece < kCpy ? piece : 0], cp_soff);
    else if (piece < 2 * kCpy) copy16_to_lds(yrs, dst + kOffY + (piece - kCpy) * 1024, cvoff[piece < 2 * kCpy ? piece - kCpy : 0], cp_soff);
    else if (!DQ)
      copy4_to_lds(ldrs, lds_base + stage * kStageBytes + ((wave & 1) ? kOffDelta : kOffLse), lane * 4, cp_ld_soff);
  };

  // row-major operand reads (A of T1 / T2): lane (ln, hf) reads chunk 2 kk + hf of row 32 mb + ln
  int rm_rd[8];                                       // + mb * 8192
#pragma unroll
  for (int kk = 0; kk < 8; ++kk) rm_rd[kk] = ln * 256 + (((2 * kk + hf) ^ lds_row_swizzle(ln)) << 4);
  // transposed operand reads (A of the second MFMAs) for head-dim block db and k-step (mb, j2): the lane's
  // 8 streamed rows are R + {0..3} and R + 8 + {0..3}, R = 32 mb + 16 j2 + 4 hf -- the rows its P / dS
  // registers hold.  One ds_read_b64_tr_b16 per group of 4 rows: within 16 lanes, lane s supplies the
  // address of row R + s/4, head-dim values 4 (s%4) .. +3 of the 16-column strip, and receives column s.
  int tr_rd[4][2];                                    // [db][second four rows]  + mb * 8192 + j2 * 4096
  {
    const int s16 = lane & 15, strip = (lane >> 4) & 1;
    const int cl = 2 * strip + ((s16 & 3) >> 1);
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int row = 8 * h + 4 * hf + (s16 >> 2);
        tr_rd[db][h] = row * 256 + (((4 * db + cl) ^ lds_row_swizzle(row)) << 4) + (s16 & 1) * 8;
      }
  }
  typedef __attribute__((address_space(3))) bf16x4* lds_bf16x4;
  f32x16 acc1[4], acc2[4];      // DQ: acc1 = dQ^T.  Otherwise acc1 = dK^T, acc2 = dV^T
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) { acc1[i][j] = 0.f; acc2[i][j] = 0.f; }
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // Tile t lives in stage t % 4 and is processed as two halves of 32 streamed rows.  Per tile the matrix
  // pipe sees one unbroken sequence of MFMA slots in four phases:
  //   P0  T1 / T2 of (t, second half)      16 slots, each carrying P / dS of one register of (t, first half)
  //   P1  accumulate (t, first half)       16 slots (8 for dQ)
  //   P2  T1 / T2 of (t+1, first half)     16 slots, each carrying P / dS of one register of (t, second half)
  //   P3  accumulate (t, second half)      16 slots (8 for dQ)
  // The LDS operand of slot s+4 is read in slot s, across phase and tile boundaries, so the pipe never
  // waits for LDS at the start of a phase.  An iteration starts by waiting for this wavefront's copies of
  // tile t+1 (those of tile t+2 stay in flight) and a barrier, after which tile t+1 is complete for every
  // wavefront and nobody reads tile t-1 any more, whose stage then receives tile t+3.  Tiles past the end
  // are copied as zeros (and their T1 / T2 computed, unused) so that the number of copies in flight
  // stays the same.
  // operand reads in flight ahead of the MFMAs (2, 4 and 8 measure the same; 2 keeps the dQ pass inside 256 registers)
  constexpr int kDepth = DQ ? 2 : 4;
  constexpr int kAcc = DQ ? 8 : 16;                        // slots of an accumulate phase
  constexpr int kP1 = 16, kP2 = 16 + kAcc, kP3 = 32 + kAcc, kSlots = 32 + 2 * kAcc;
  typedef __attribute__((address_space(3))) const bf16x8* lds_bf16x8;
  typedef __attribute__((address_space(3))) const f32x4* lds_f32x4;
  // LDS addresses of the operand reads.  rm_a / tr_a hold, per lane, the addresses inside ONE tile's stage and are
  // moved on to the next stage in place, each at a point of the slot sequence where no read of its kind is due
  // (rm_a in the last kDepth slots of P0: the reads of the current tile's T1 / T2 operands are all issued by then and
  // those of the next tile start at slot kP2 - kDepth; tr_a in the last kDepth slots, after the last transposed read).
  // ld_cur / ld_next address lse2 / -delta of the current and the next tile.  Everything else about an address
  // is an immediate offset of the LDS instruction.
  int rm_a[8], tr_a[4][2];
#pragma unroll
  for (int kk = 0; kk < 8; ++kk) rm_a[kk] = rm_rd[kk] + (int)lds_base;
#pragma unroll
  for (int db = 0; db < 4; ++db) { tr_a[db][0] = tr_rd[db][0] + (int)lds_base; tr_a[db][1] = tr_rd[db][1] + (int)lds_base; }
  int ld_cur = (int)lds_base + hf * 16, ld_next = ld_cur + kStageBytes;
  // slot i (0..15) of the T1 / T2 sequence of one half: k-step i / 2, X (T1) on even and Y (T2) on odd slots
  auto read_rm = [&](int mb, int i) -> bf16x8 {
    return *(lds_bf16x8)(uintptr_t)(uint32_t)(rm_a[i >> 1] + mb * 8192 + ((i & 1) ? kOffY : 0));
  };
  // T2 starts from -delta of the half's streamed rows (dQ pass: of this lane's stationary row), so that what
  // the vector unit receives is dP - delta already
  f32x16 nd;
  auto t_mfma = [&](int i, const bf16x8& a, f32x16& n1, f32x16& n2) {
    const int kk = i >> 1;
    if (i & 1) n2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, yf[kk], kk == 0 ? nd : n2, 0, 0, 0);
    else n1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, xf[kk], kk == 0 ? zero : n1, 0, 0, 0);
  };
  // slot i of an accumulate phase of half mb: head-dim block and k-step, X^T (dS) / Y^T (P) alternating for dK, dV
  auto read_acc = [&](int mb, int i) -> bf16x8 {
    const int m = DQ ? i : (i >> 1);
    const int off = mb * 8192 + (m >> 2) * 4096 + ((!DQ && (i & 1)) ? kOffY : 0);
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4)(uintptr_t)(uint32_t)(tr_a[m & 3][0] + off));
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4)(uintptr_t)(uint32_t)(tr_a[m & 3][1] + off));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  bf16x8 pfrag[2], dsfrag[2];     // P and dS of the half being accumulated as B operands (two k-steps)
  bf16x8 ring[kDepth];
  f32x16 ta1, ta2, tb1, tb2;      // T1 / T2 of the two halves in flight: (t, first half), (t, second half)
  f32x4 lv[5];                    // lse2 of 4 streamed rows per entry (dK / dV pass), read one group ahead

  // Hidden elements (rows past the end of the streamed tensor, the causal mask) get a score of -inf,
  // hence P = dS = 0.  Only the last tile of a head and the tiles the diagonal crosses need it.
  auto mask_half = [&](f32x16& c1, int cb) {
    bool need_mask = cb + 32 > n_str;
    if (CAUSAL) need_mask = need_mask || (DQ ? (cb + 31 > r0 + shift) : (r0 + kRowsPerWg - 1 > cb + shift));
    if (need_mask) {
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int c = cb + (j >> 2) * 8 + hf * 4 + (j & 3);     // streamed row of this element
        bool hidden = c >= n_str;
        if (CAUSAL) hidden = hidden || (DQ ? (c > my_r + shift) : (my_r > c + shift));
        if (hidden) c1[j] = -INFINITY;
      }
    }
  };
  // lse2 of rows 8 g + 4 hf .. + 3 of half mb of the current (next: of the following) tile
  auto read_ld = [&](bool next, int mb, int g, f32x4& l) {
    l = *(lds_f32x4)(uintptr_t)(uint32_t)((next ? ld_next : ld_cur) + kOffLse + (mb * 32 + g * 8) * 4);
  };
  // -delta of rows 8 g + 4 hf .. + 3 (g = 0..3) of half mb of the current / following tile, in the order of the
  // accumulator registers of T2 (dK / dV pass), one group per call
  auto read_nd = [&](bool next, int mb, int g) {
    const f32x4 d = *(lds_f32x4)(uintptr_t)(uint32_t)((next ? ld_next : ld_cur) + kOffDelta + (mb * 32 + g * 8) * 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) nd[4 * g + e] = d[e];
  };
  // P / dS of the half in (c1, c2): 16 accumulator registers, spread over the 16 slots in which the next
  // half's T1 / T2 are issued AND the first slots of the accumulate phase that follows (a wavefront issues
  // one vector instruction every ~5 cycles, so 16 slots of 32 cycles do not hold all of it).  Register e
  // enters at slot first_slot(e); its work is a three-stage pipeline so that no instruction waits for the
  // one issued just before it:
  //   first_slot      argument of the exponential
  //   first_slot + 1  exponential
  //   first_slot + 2  dS = P (dP - delta)     (c2 arrives as dP - delta)
  // Registers 0-7 (k-step 0 of the accumulate phase) are packed before that phase starts, registers 8-15
  // before its second half does.
  auto first_slot = [](int e) -> int {
    if (DQ) return e < 8 ? (e * 3) / 2 : 1 + e;          // 0,1,3,4,6,7,9,10 | 9..16: packed at slots 13 and 19 (acc 16-19, 20-23)
    return e < 8 ? (e * 7) / 4 : 5 + e;                  // 0,1,3,5,7,8,10,12 | 13..20: packed at slots 15 and 23 (acc 16-23, 24-31)
  };
  float earg[16];
  auto vector_slot = [&](int s, f32x16& c1, f32x16& c2, int mb) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int f = first_slot(e);
      if (s == f) {
        const float l = DQ ? lse2_lane : lv[e >> 2][e & 3];
        earg[e] = __builtin_fmaf(c1[e], p.scale_log2, -l);
        // lse2 of the next four rows, one group ahead
        if (!DQ && (e & 3) == 0 && e < 12) read_ld(false, mb, (e >> 2) + 1, lv[(e >> 2) + 1]);
      }
      if (s == f + 1) c1[e] = fast_exp2(earg[e]);
      if (s == f + 2) c2[e] = c1[e] * c2[e];
    }
#pragma unroll
    for (int j2 = 0; j2 < 2; ++j2)
      if (s == first_slot(8 * j2 + 7) + 3) {
        u32x4 wp, wd;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          wp[e] = pack_bf16(c1[8 * j2 + 2 * e], c1[8 * j2 + 2 * e + 1]);
          wd[e] = pack_bf16(c2[8 * j2 + 2 * e], c2[8 * j2 + 2 * e + 1]);
        }
        pfrag[j2] = __builtin_bit_cast(bf16x8, wp);
        dsfrag[j2] = __builtin_bit_cast(bf16x8, wd);
      }
  };
  constexpr int kVecTail = DQ ? 4 : 8;      // accumulate-phase slots that still carry vector work
  auto acc_mfma = [&](int i, const bf16x8& a) {
    const int m = DQ ? i : (i >> 1);
    const int db = m & 3, j2 = m >> 2;
    if (DQ || !(i & 1)) acc1[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, dsfrag[j2], acc1[db], 0, 0, 0);
    else acc2[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pfrag[j2], acc2[db], 0, 0, 0);
  };
  // LDS operand of slot s of the current tile's sequence; s >= kSlots continues into the next tile's P0.  The
  // T1 / T2 operands of slots kP2 .. kP3 - 1 and from kSlots on belong to the next tile: rm_a has moved on by then.
  auto read_slot = [&](int s) -> bf16x8 {
    if (s >= kSlots) return read_rm(1, s - kSlots);
    if (s < kP1) return read_rm(1, s);
    if (s < kP2) return read_acc(0, s - kP1);
    if (s < kP3) return read_rm(0, s - kP2);
    return read_acc(1, s - kP3);
  };
  static_assert(kP2 - kDepth >= 16 && 4 % kDepth == 0, "rm_a moves in the last kDepth slots of P0, tr_a in the last kDepth slots of P3");

  if (ntiles > 0) {
    copy_tile(0, 0);
    copy_tile(1, 1);
    copy_tile(2, 2);
  }
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
      if (ks * 16 + hf * 8 < p.D) {
        xf[ks] = *reinterpret_cast<const bf16x8*>(xp + ks * 16);
        yf[ks] = *reinterpret_cast<const bf16x8*>(yp + ks * 16);
      } else {                                       // columns past the head dimension
        xf[ks] = bf16x8{};
        yf[ks] = bf16x8{};
      }
    }
    // Pin the loads here (the copies are invisible to the compiler's wait counting).  The dK / dV pass keeps these
    // MFMA operands in accumulation registers: its arithmetic registers are needed for the tiles of T1 / T2 that
    // the vector unit works on.  The dQ pass at two wavefronts per SIMD uses no accumulation registers at all (a
    // kernel that does gets its 256 registers split 128 / 128).
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      if (DQ) { asm volatile("" : "+v"(xf[ks])); asm volatile("" : "+v"(yf[ks])); }
      else { asm volatile("" : "+a"(xf[ks])); asm volatile("" : "+a"(yf[ks])); }
    }
    if (DQ) {
      // This pass runs first and prepares what both passes need per query row: delta = rowsum(dout * out), kept
      // negated (the dP products start from it), and lse2 = lse * log2(e) with -inf (a row that saw no key) turned
      // into +inf so that P = exp2(s - lse2) = 0 there.  The lane pair (l, l ^ 32) holds the two halves of the
      // row's dout; the matching halves of out are read here once.
      const uint16_t* op = p.out + b * p.o_sb + (int64_t)row * p.o_ss + hs * p.o_sh + hf * 8;
      float part = 0.f;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        if (ks * 16 + hf * 8 < p.D) {
          const bf16x8 o8 = *reinterpret_cast<const bf16x8*>(op + ks * 16);
#pragma unroll
          for (int j = 0; j < 8; ++j) part = __builtin_fmaf((float)yf[ks][j], (float)o8[j], part);
        }
      }
      const float delta = pair_sum(part);
      const int64_t r = ((int64_t)b * p.Hq + hs) * p.Sq + row;
      const float l = p.lse[r];
      lse2_lane = (l == -INFINITY) ? INFINITY : l * kLog2e;
      delta_lane = -delta;
      if (hf == 0 && my_r < n_st) {
        p.delta[r] = delta_lane;
        p.lse2[r] = lse2_lane;
        if (p.softmax_d) p.softmax_d[r] = delta;     // for callers that want flash-attn's softmax_d back
      }
    }
    asm volatile("" : "+v"(lse2_lane), "+v"(delta_lane));
  }
  if (ntiles > 0) {
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * kCopiesPerTile) : "memory");      // two tiles of copies may stay in flight
    __builtin_amdgcn_s_barrier();
    if (DQ) {
#pragma unroll
      for (int j = 0; j < 16; ++j) nd[j] = delta_lane;
    } else {
#pragma unroll
      for (int g = 0; g < 4; ++g) read_nd(false, 0, g);
    }
    // T1 / T2 of the first half of tile 0, nothing to interleave with
#pragma unroll
    for (int i = 0; i < kDepth; ++i) ring[i] = read_rm(0, i);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      t_mfma(i, ring[i % kDepth], ta1, ta2);
      if (i + kDepth < 16) ring[i % kDepth] = read_rm(0, i + kDepth);
    }
#pragma unroll
    for (int i = 0; i < kDepth; ++i) ring[i] = read_rm(1, i);            // slots 0 .. 3 of tile 0
    if (!DQ) {
      read_ld(false, 0, 0, lv[0]);
#pragma unroll
      for (int g = 0; g < 4; ++g) read_nd(false, 1, g);        // for T2 of the second half, first thing in the loop
    }
  }
  int cur_r = 0;                                         // t % span
  for (int t = 0; t < ntiles; ++t) {
    const int c0 = (first_tile + cur_r) * kTile;
    if (++cur_r == span) cur_r = 0;                      // (t + 1) % span
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kCopiesPerTile) : "memory");          // one tile of copies stays in flight
    __builtin_amdgcn_s_barrier();
    copy_setup();
    // byte distance from this tile's stage to the next tile's, and from that one to the one after
    const int step1 = ((t + 1) & 3) == 0 ? -3 * kStageBytes : kStageBytes;
    const int step2 = ((t + 2) & 3) == 0 ? -3 * kStageBytes : kStageBytes;
    static_assert(kSlots % kDepth == 0 && 16 % kDepth == 0, "the ring position is the slot number modulo its depth");
    mask_half(ta1, c0);
#pragma unroll
    for (int i = 0; i < 16; ++i) {                       // P0, carrying the copies of tile t+3
      t_mfma(i, ring[i % kDepth], tb1, tb2);
      vector_slot(i, ta1, ta2, 0);
      if (i < kCopiesPerTile) copy_piece(i, (t + 3) & 3);
      ring[i % kDepth] = read_slot(i + kDepth);
      if (i >= 16 - kDepth) {                            // the last read of this tile's T1 / T2 operands is out: on to the next
#pragma unroll
        for (int j = 0; j < 8 / kDepth; ++j) rm_a[(i - (16 - kDepth)) * (8 / kDepth) + j] += step1;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < kAcc; ++i) {                     // P1
      if (i < kVecTail) vector_slot(16 + i, ta1, ta2, 0);
      acc_mfma(i, ring[(kP1 + i) % kDepth]);
      if (!DQ && i == kAcc - 2) read_ld(false, 1, 0, lv[0]);
      // -delta for T2 of (t+1, first half), which starts in P2: read once the vector work on this half's dP is
      // through (slot 7), so that the values can land in the registers T2 accumulates in
      if (!DQ && i >= 8 && i < 12) read_nd(true, 0, i - 8);
      ring[(kP1 + i) % kDepth] = read_slot(kP1 + i + kDepth);
      __builtin_amdgcn_sched_barrier(0);
    }
    mask_half(tb1, c0 + 32);
#pragma unroll
    for (int i = 0; i < 16; ++i) {                       // P2
      t_mfma(i, ring[(kP2 + i) % kDepth], ta1, ta2);
      vector_slot(i, tb1, tb2, 1);
      ring[(kP2 + i) % kDepth] = read_slot(kP2 + i + kDepth);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < kAcc; ++i) {                     // P3
      if (i < kVecTail) vector_slot(16 + i, tb1, tb2, 1);
      acc_mfma(i, ring[(kP3 + i) % kDepth]);
      if (!DQ && i == kAcc - 2) read_ld(true, 0, 0, lv[0]);
      if (!DQ && i >= 8 && i < 12) read_nd(true, 1, i - 8);            // T2 of (t+1, second half): P0 of the next tile
      ring[(kP3 + i) % kDepth] = read_slot(kP3 + i + kDepth);
      if (i >= kAcc - kDepth) {                          // the last transposed read of this tile has been issued
#pragma unroll
        for (int j = 0; j < 4 / kDepth; ++j) {
          const int db = (i - (kAcc - kDepth)) * (4 / kDepth) + j;
          tr_a[db][0] += step1; tr_a[db][1] += step1;
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    ld_cur = ld_next;
    ld_next += step2;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the zero-filled copies of tiles past the end

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
      if (row < n_st && chunk * 8 < p.D) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(os + r * (kOStride * 2) + chunk * 16);
        *reinterpret_cast<u32x4*>(op + (int64_t)row * d_ss) = w;
      }
    }
  };
  if (DQ) {
    write_out(acc1, p.scale, p.dq, p.dq_sb, p.dq_ss, p.dq_sh, hs);
    if (p.dq_acc != nullptr && my_r < n_st) {
      // fp32 accumulator (B, Sq, Hq, D) contiguous; every element belongs to exactly one lane
      float* ap = p.dq_acc + (((int64_t)b * p.Sq + my_r) * p.Hq + hs) * p.D;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          if (db * 32 + g * 8 + hf * 4 < p.D) {
            f32x4* a4 = reinterpret_cast<f32x4*>(ap + db * 32 + g * 8 + hf * 4);
            f32x4 v = *a4;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += acc1[db][4 * g + e] * p.scale;
            *a4 = v;
          }
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
  // -delta, lse2 and delta, (B, Hq, Sq) fp32 each, every one starting on a 16-byte boundary
  return ((((int64_t)B * Hq * Sq + 3) & ~int64_t(3)) * 3) * 4;
}

// Scratch of the entry point that allocates nothing: delta and lse2 of up to kScratchRows (batch, head, row)
// triples.  Every GPU the library runs on holds its own copy until the process ends.
constexpr int64_t kScratchRows = int64_t(1) << 20;
static __device__ __align__(256) unsigned char scratch[kScratchRows * 8 + 32];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device.  In host code the array's name is only a handle for
// the runtime: the address a kernel can use comes from hipGetSymbolAddress, once per device.
int scratch_address(void** ptr) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MHIP_ERUNTIME;
  void* cached = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (cached == nullptr) {
    void* fresh = nullptr;
    if (hipGetSymbolAddress(&fresh, HIP_SYMBOL(scratch)) != hipSuccess || fresh == nullptr) {
      (void)hipGetLastError();
      return MHIP_ERUNTIME;
    }
    g_scratch_ptr[dev].store(fresh, std::memory_order_release);   // every thread would store the same address
    cached = fresh;
  }
  *ptr = cached;
  return MHIP_OK;
}

// own_scratch: take the workspace from `scratch` (resolved after the arguments have been checked)
int bwd_block(const void* dout, const void* q, const void* k, const void* v,
              const void* out, const float* lse,
              void* dq, void* dk, void* dv, float* dq_acc,
              int B, int Sq, int Sc, int Hq, int Hkv, int D,
              int64_t q_sb, int64_t q_ss, int64_t q_sh,
              int64_t k_sb, int64_t k_ss, int64_t k_sh,
              int64_t dk_sb, int64_t dk_ss, int64_t dk_sh,
              int64_t dq_sb, int64_t dq_ss, int64_t dq_sh,
              int64_t o_sb, int64_t o_ss, int64_t o_sh,
              float softmax_scale, int mask, void* workspace, bool own_scratch, hipStream_t st) {
  if (B < 0 || Sq < 0 || Sc < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return MHIP_EINVAL;
  if (!(softmax_scale > 0.f) || !(softmax_scale < INFINITY)) return MHIP_EINVAL;
  if (mask != MHIP_MASK_NONE && mask != MHIP_MASK_CAUSAL) return MHIP_EINVAL;
  if (D < 8 || D > kD || (D & 7) != 0) return MHIP_EHEADDIM;     // below 128 the missing columns are zeros on chip
  if (B == 0) return MHIP_OK;
  if (Sq > 0 && (!dout || !q || !out || !lse || !dq || (!workspace && !own_scratch))) return MHIP_EINVAL;
  if (Sc > 0 && (!k || !v || !dk || !dv)) return MHIP_EINVAL;
  const void* ptrs[] = {dout, q, k, v, out, dq, dk, dv, workspace, dq_acc};
  for (const void* ptr : ptrs)
    if (ptr && !aligned16(ptr)) return MHIP_EALIGN;
  const int64_t strides[] = {q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, dk_sb, dk_ss, dk_sh, dq_sb, dq_ss, dq_sh,
                             o_sb, o_ss, o_sh};
  for (int64_t s : strides)
    if (s < 0 || (s & 7)) return MHIP_EALIGN;
  // streamed tiles are fetched through 32-bit buffer offsets
  const int64_t q_span = ((int64_t)Sq * q_ss + (int64_t)Hq * q_sh) * 2;
  const int64_t k_span = (int64_t)Sc * k_ss * 2;
  if (q_span >= (int64_t(1) << 31) || k_span >= (int64_t(1) << 31)) return MHIP_EUNSUPPORTED;
  if ((int64_t)B * Hq * Sq >= (int64_t(1) << 30)) return MHIP_EUNSUPPORTED;     // lse2 / delta are addressed with 32-bit byte offsets
  // below 128 the lanes of the missing columns carry the offset kNoColumn, which has to be out of range
  if (D < kD && (q_span >= (int64_t(1) << 30) || k_span >= (int64_t(1) << 30))) return MHIP_EUNSUPPORTED;
  if (own_scratch && Sq > 0) {
    if ((int64_t)B * Hq * Sq > kScratchRows) return MHIP_ETOOLARGE;
    const int rc = scratch_address(&workspace);
    if (rc != MHIP_OK) return rc;
  }

  BwdParams p;
  p.q = static_cast<const uint16_t*>(q); p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v); p.dout = static_cast<const uint16_t*>(dout);
  float* delta_buf = static_cast<float*>(workspace);
  const int64_t slot = ((int64_t)B * Hq * Sq + 3) & ~int64_t(3);                // 16-byte aligned
  float* lse2_buf = delta_buf + slot;
  float* softmax_d = own_scratch ? nullptr : lse2_buf + slot;      // the built-in scratch has no room for it
  p.lse2 = lse2_buf; p.delta = delta_buf; p.softmax_d = softmax_d;
  p.out = static_cast<const uint16_t*>(out); p.lse = lse;
  p.dq = static_cast<uint16_t*>(dq); p.dk = static_cast<uint16_t*>(dk); p.dv = static_cast<uint16_t*>(dv);
  p.dq_acc = dq_acc;
  p.B = B; p.Sq = Sq; p.Sc = Sc; p.Hq = Hq; p.Hkv = Hkv; p.group = Hq / Hkv;
  p.D = D;
  p.q_sb = q_sb; p.q_ss = q_ss; p.q_sh = q_sh;
  p.k_sb = k_sb; p.k_ss = k_ss; p.k_sh = k_sh;
  p.dk_sb = dk_sb; p.dk_ss = dk_ss; p.dk_sh = dk_sh;
  p.dq_sb = dq_sb; p.dq_ss = dq_ss; p.dq_sh = dq_sh;
  p.o_sb = o_sb; p.o_ss = o_ss; p.o_sh = o_sh;
  p.scale = softmax_scale; p.scale_log2 = softmax_scale * kLog2e;
  const bool causal = mask == MHIP_MASK_CAUSAL;

  if (Sq > 0) {
    // dQ (and delta / lse2 for both passes): one workgroup per 256 query rows; has to run before the dK / dV pass
    p.n_tiles = (Sq + kRowsQ - 1) / kRowsQ;
    p.total = B * Hq * p.n_tiles;
    p.per_xcd = (p.total + 7) / 8;
    p.heads_per_xcd = (B * Hq) % 8 == 0 ? (B * Hq) / 8 : 0;
    if (causal) hipLaunchKernelGGL((bwd_main<true, true>), dim3(p.per_xcd * 8), dim3(512), 0, st, p);
    else hipLaunchKernelGGL((bwd_main<true, false>), dim3(p.per_xcd * 8), dim3(512), 0, st, p);
  }
  if (Sc > 0) {
    // dK, dV: one workgroup per 128 keys of one kv head
    p.n_tiles = (Sc + kRowsKv - 1) / kRowsKv;
    p.total = B * Hkv * p.n_tiles;
    p.per_xcd = (p.total + 7) / 8;
    p.heads_per_xcd = (B * Hkv) % 8 == 0 ? (B * Hkv) / 8 : 0;
    if (causal) hipLaunchKernelGGL((bwd_main<false, true>), dim3(p.per_xcd * 8), dim3(256), 0, st, p);
    else hipLaunchKernelGGL((bwd_main<false, false>), dim3(p.per_xcd * 8), dim3(256), 0, st, p);
  }
  return launch_status();
}
}  // namespace

// Resolves, for the current device, whatever the entry points otherwise look up on their first call (the address
// of the built-in scratch): a caller that records its calls (HIP graph capture) makes this call first, outside
// the capture.
extern "C" int mhip_init(void) {
  void* unused = nullptr;
  return scratch_address(&unused);
}

extern "C" int mhip_attn_bwd_block(const void* dout, const void* q, const void* k, const void* v,
                                   const void* out, const float* lse,
                                   void* dq, void* dk, void* dv, float* dq_acc,
                                   int B, int Sq, int Sc, int Hq, int Hkv, int D,
                                   int64_t q_sb, int64_t q_ss, int64_t q_sh,
                                   int64_t k_sb, int64_t k_ss, int64_t k_sh,
                                   int64_t dk_sb, int64_t dk_ss, int64_t dk_sh,
                                   int64_t dq_sb, int64_t dq_ss, int64_t dq_sh,
                                   int64_t o_sb, int64_t o_ss, int64_t o_sh,
                                   float softmax_scale, int mask, int deterministic,
                                   void* workspace, void* stream) {
  (void)deterministic;   // there are no atomics: every run is deterministic
  return bwd_block(dout, q, k, v, out, lse, dq, dk, dv, dq_acc, B, Sq, Sc, Hq, Hkv, D, q_sb, q_ss, q_sh,
                   k_sb, k_ss, k_sh, dk_sb, dk_ss, dk_sh, dq_sb, dq_ss, dq_sh, o_sb, o_ss, o_sh, softmax_scale, mask,
                   workspace, false,
                   static_cast<hipStream_t>(stream));
}

extern "C" int mhip_attn_bwd_block_noalloc(const void* dout, const void* q, const void* k, const void* v,
                                           const void* out, const float* lse,
                                           void* dq, void* dk, void* dv, float* dq_acc,
                                           int B, int Sq, int Sc, int Hq, int Hkv, int D,
                                           int64_t q_sb, int64_t q_ss, int64_t q_sh,
                                           int64_t k_sb, int64_t k_ss, int64_t k_sh,
                                           int64_t dk_sb, int64_t dk_ss, int64_t dk_sh,
                                           int64_t dq_sb, int64_t dq_ss, int64_t dq_sh,
                                           int64_t o_sb, int64_t o_ss, int64_t o_sh,
                                           float softmax_scale, int mask, int deterministic, void* stream) {
  (void)deterministic;
  // the dQ pass overwrites the part of the scratch the dK / dV pass reads, so nothing has to be cleared
  return bwd_block(dout, q, k, v, out, lse, dq, dk, dv, dq_acc, B, Sq, Sc, Hq, Hkv, D, q_sb, q_ss, q_sh,
                   k_sb, k_ss, k_sh, dk_sb, dk_ss, dk_sh, dq_sb, dq_ss, dq_sh, o_sb, o_ss, o_sh, softmax_scale, mask,
                   nullptr, true,
                   static_cast<hipStream_t>(stream));
}
