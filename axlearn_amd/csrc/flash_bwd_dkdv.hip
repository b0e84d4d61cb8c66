// dK / dV kernel of the flash-attention backward for gfx950 (bf16).
//
// Replaces axlearn/common/flash_attention/gpu_attention.py:436-528 (`_mha_backward_kernel_dkdv`):
//   p = exp(qk - lse); dv += p^T dO; dp = dO v^T; ds = p * (dp - delta) * scale; dk += ds^T q,
// with p and ds rounded to bf16 before their GEMMs and fp32 accumulation (:513, :518).
//
// Mapping.  A workgroup owns 128 keys of one (batch, kv head); each of its 4 wavefronts keeps the
// K and V fragments of 32 keys in registers (B operands) and the fp32 dK^T / dV^T accumulators of
// those keys (128 registers), and loops over ALL query heads of the kv head's group and all query
// tiles that can see the keys, so dK/dV need neither atomics nor a pass that sums repeated KV
// heads.  Query tiles (32 rows of Q and dO plus their scaled lse / delta / segment ids) stream
// through a six-deep LDS ring, filled by direct global->LDS loads: no staging registers and no LDS
// store instructions, one unpadded XOR-swizzled copy per tile that serves both the row-per-lane
// fragment reads of stage A and the transposing reads of stage B without bank conflicts.
//
// Register pressure allows one wavefront per SIMD, so nobody else can cover this wavefront's
// latencies; the loop is software pipelined by hand instead, with three tiles in flight.  Iteration j
// runs
//   stage A of tile j+2:      S = Q K^T and dP = dO V^T   (2*D/16 MFMAs, lane = key, registers = queries)
//   elementwise of tile j+1:  P = exp2(S*c - lse), dS = P * (dP - delta), packed to 16 bits
//   stage B of tile j:        dV^T += dO^T P and dK^T += Q^T dS   (D/4 MFMAs, A operands from
//                             transposing LDS reads of the same dO / Q tiles)
// while tile j+3 is awaited and tiles j+4, j+5 are in flight from HBM / L2.  Everything that is not
// an MFMA is dealt out over the MFMA slots of the iteration.  Tiles that no mask touches run a copy
// of the loop without mask arithmetic; the choice is made per run of tiles, never inside an iteration
// (a branch would end the scheduling region).
#include <type_traits>

#include "flash_bwd.h"

#ifndef AXL_DKDV_PG
#define AXL_DKDV_PG 2
#endif

namespace axl {

template <int D>
struct DkvTile {
  static constexpr int BKV = 128;            // keys per workgroup (32 per wavefront)
  static constexpr int BQ = 32;              // query rows per LDS tile
  static constexpr int ROWB = D * 2;         // bytes per row: unpadded, chunks swizzled (tile_swizzle)
  static constexpr int TILE_BYTES = BQ * ROWB;                   // Q tile, then the dO tile
  static constexpr int STAT_BASE = 2 * TILE_BYTES;
  static constexpr int STAT_BYTES = 4 * BQ * 4;  // -lse*log2e | -delta | segment id | (unused) per query row
  static constexpr int BUF_BYTES = STAT_BASE + STAT_BYTES;
  static constexpr int NBUF = 6;
  static constexpr int RPI = 1024 / ROWB;                        // rows per direct-to-LDS instruction
  static constexpr int DMA_PER_WAVE = BQ / 4 / RPI;              // per tensor per tile (8 rows per wavefront)
  static constexpr int DMA_PER_TILE = 2 * DMA_PER_WAVE + 1;      // Q, dO and one row of statistics
  static constexpr int LDS_BYTES = NBUF * BUF_BYTES;
};

constexpr int kMaxSubDkv = 1024;                 // query tiles whose segment ids the dK/dV kernel classifies
constexpr int kNotUniformDkv = -0x7fffffff - 1;  // marks a tile with more than one segment id

// SPILL: the kernel also stores every tile's dS (rounded to the input dtype, as it enters the dK
// product) into the a.ds workspace, for the streaming dQ kernel.  Causal or sliding-window mask with
// q_off 0 and T == S; masked elements are stored as the zeros they are.
template <typename E, int D, bool HAS_SEG, int AUX, bool SPILL = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void flash_bwd_dkdv_kernel(const BwdArgs a) {
  static_assert(!SPILL || !AUX, "the spill path has no bias or dropout mask");
  using Tile = DkvTile<D>;
  constexpr bool HAS_BIAS = (AUX & (kAuxBias16 | kAuxBias32)) != 0, BIAS_F32 = (AUX & kAuxBias32) != 0;
  constexpr bool HAS_DROP = (AUX & kAuxDrop) != 0;
  constexpr int KK = D / 16, DT = D / 32;
  constexpr int NA = 2 * KK;          // stage-A MFMAs per tile
  constexpr int NB = 4 * DT;          // stage-B MFMAs per tile
  static_assert(Tile::BQ == 32, "tiling");
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int G = a.Hq / a.Hkv;
  // blockIdx -> (key block, batch, kv head).  When the (batch, kv head) pairs divide evenly over the
  // 8 XCDs (workgroup i is dispatched to XCD i % 8), an XCD works through one pair after the other,
  // so the workgroups that run together stream the same Q / dO rows through that XCD's L2; within a
  // pair the earliest key blocks (most queries under a causal mask) come first.
  // With a.kb_per_wg == 2 a workgroup works through TWO key blocks of its pair, one after the other:
  // block kb0 of the first half and its mirror image nkb - 1 - kb0.  Under a causal mask the two see
  // complementary shares of the queries, so every workgroup of the launch walks the same number of
  // tiles: the workgroups of a pair that start together stay in step down their first blocks (one of
  // them brings a Q / dO tile into L2, the others find it there), half as many workgroups start and
  // end, and the launch divides evenly over the CUs.
  const int npairs = a.B * a.Hkv, nkb = a.S / Tile::BKV;
  const int nkb_wg = nkb / a.kb_per_wg;              // key blocks the blockIdx mapping numbers
  int kb0, pair;
  if (npairs % 8 == 0) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int ppx = npairs >> 3;                     // pairs per XCD
    const int grp = slot / (AXL_DKDV_PG * nkb_wg);   // group of AXL_DKDV_PG pairs worked through together
    const int r = slot - grp * (AXL_DKDV_PG * nkb_wg);
    const int pg = min(AXL_DKDV_PG, ppx - grp * AXL_DKDV_PG);
    pair = xcd + 8 * (grp * AXL_DKDV_PG + r % pg);
    kb0 = r / pg;
  } else {
    kb0 = blockIdx.x / npairs;
    pair = blockIdx.x % npairs;
  }
  const int b = pair / a.Hkv, hk = pair % a.Hkv;
  for (int pass = 0; pass < a.kb_per_wg; pass++) {
  // Everything a key block needs is derived again from the thread index inside its pass (the empty
  // statement hides the index's origin from the compiler): hoisted out of the pass loop, the lane
  // offsets of the prologue and the epilogue would stay live through the main loops, which have no
  // register to spare.
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  const int kb = pass == 0 ? kb0 : nkb - 1 - kb0;
  const int k0_wg = kb * Tile::BKV;
  const int k0 = k0_wg + wave * 32;  // this wavefront's keys

  // K and V fragments (B operands): lane (key l32, k-group g) holds d = 16kk + 8g .. +7.
  const __bf16* kp = (const __bf16*)a.k + b * a.ks.b + (int64_t)(k0 + l32) * a.ks.s + hk * a.ks.h;
  const __bf16* vp = (const __bf16*)a.v + b * a.vs.b + (int64_t)(k0 + l32) * a.vs.s + hk * a.vs.h;
  bf16x8 kf[KK], vf[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) {
    kf[kk] = load8_within(kp, 16 * kk + 8 * g, a.d_real);
    vf[kk] = load8_within(vp, 16 * kk + 8 * g, a.d_real);
  }
  const int kpos = k0 + l32;
  int seg_k = 0;
  if (HAS_SEG) seg_k = a.seg[(int64_t)b * a.T + k0 + l32];

  // Query rows that can see any key of this workgroup.
  int q_begin = 0, q_end = a.T;
  if (a.mask_kind != AXL_MASK_NONE) {
    q_begin = max(0, k0_wg - a.q_off);
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW)
      q_end = min(a.T, k0_wg + Tile::BKV - 1 + a.window - a.q_off + 1);
  }
  // With segment ids: the query range shrinks to the hull of the 32-row groups that hold an id
  // between the smallest and the largest id of this workgroup's keys, and s_sub records for every query
  // tile from sub_g0 on whether its rows carry a single id (both from the table of per-group id ranges
  // that a small kernel leaves in the workspace).
  __shared__ int s_sub[HAS_SEG && !AUX ? kMaxSubDkv : 1];
  int sub_g0 = 0;
  if (HAS_SEG)
    sub_g0 = classify_segment_groups_tbl<256>(a.seg_tbl + (int64_t)b * (a.T / kSegGroupRows), k0_wg / kSegGroupRows,
                                              Tile::BKV / kSegGroupRows, tid, q_begin, q_end, s_sub,
                                              AUX ? 0 : kMaxSubDkv, kNotUniformDkv);
  const int t_begin = q_begin / Tile::BQ;
  const int nt = max(0, (q_end + Tile::BQ - 1) / Tile::BQ - t_begin);
  if constexpr (SPILL) {
    // which tiles' dS this key block stores, for the streaming dQ kernel (the same for every kv head)
    if (a.kb_tbl && hk == 0 && tid == 0) a.kb_tbl[b * nkb + kb] = make_int2(t_begin, t_begin + nt);
  }
  // Tiles in processing order: query tile (outer, from the LAST one down to the diagonal) x query head
  // (inner).  Every workgroup of a (batch, kv head) pair starts at the same last tile and walks down
  // until it reaches its own diagonal, so the workgroups that run together read the same Q / dO rows
  // at the same time and all but one of them find them in L2.  The second key block of a workgroup is
  // walked the other way, from its diagonal UP to the last tile: a workgroup that took nkb - kb0
  // steps down its first block starts its second at tile nkb - 1 - kb0, so at any moment the
  // workgroups that started together are again all at the same tile, and they end together.
  const int total = nt * G;
  const int dir = pass == 0 ? -1 : 1;
  const int t_first = t_begin + (dir < 0 ? max(nt - 1, 0) : 0);  // the tile the sequence starts with
  // dS store cursor (SPILL): block of this wavefront's 32 keys in the run of the tile whose stage B
  // the iteration executes; it walks the tiles in processing order.  A lane stores its two packed
  // operand registers at [query half][key l32][8 g .. 8 g + 7].
  char* ds_ptr = nullptr;
  int st_t = t_first, st_h = 0;
  const unsigned ds_lane = (unsigned)(l32 * 32 + g * 16);
  if constexpr (SPILL)
    ds_ptr = (char*)a.ds + (ds_run_start(pair, a.T, G, t_first, 0) + 4 * kb + wave) * kDsBlockBytes;
  // keep(q, k)  <=>  (unsigned)(qpos - kpos) <= limit
  const unsigned limit = a.mask_kind == AXL_MASK_NONE             ? 0xffffffffu
                         : a.mask_kind == AXL_MASK_SLIDING_WINDOW ? (unsigned)a.window
                                                                  : 0x7fffffffu;

  floatx16 dk_acc[DT], dv_acc[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dk_acc[i][r] = dv_acc[i][r] = 0.f;
  const float c = a.scale * kLog2e;

  // ---- tile loads: direct global->LDS, 1 KB (RPI rows) per instruction.  Wavefront w fetches rows
  // 8w .. 8w+7 of the Q and of the dO tile; lane l fills chunk slot l % CPR of row l / CPR with the
  // global chunk that the swizzle puts there.  Lanes 0..7 of wavefront w also fetch one row of
  // statistics (4 query rows each): w = 0 the scaled lse, 1 delta, 2 the segment ids.
  constexpr int CPR = D / 8;  // 16-byte chunks per row
  constexpr bool PAIRS = Tile::DMA_PER_WAVE == 2;  // the two loads of a tensor go out as one pair
  static_assert(Tile::DMA_PER_WAVE <= 2, "tile loads per tensor");
  unsigned q_lane[Tile::DMA_PER_WAVE], d_lane[Tile::DMA_PER_WAVE];  // byte offsets from the tile's first row
#pragma unroll
  for (int i = 0; i < Tile::DMA_PER_WAVE; i++) {
    const int row = 8 * wave + Tile::RPI * i + lane / CPR;
    const int slot_chunk = (lane % CPR) ^ tile_swizzle<D>(row);
    const int chunk = slot_chunk * 8 < a.d_real ? slot_chunk : 0;
    // the second load of a pair carries an instruction offset of 1024, which also moves its source
    q_lane[i] = (unsigned)(row * (int)a.qs.s + chunk * 8) * 2 - (i % 2) * 1024;
    d_lane[i] = (unsigned)(row * (int)a.dos.s + chunk * 8) * 2 - (i % 2) * 1024;
  }
  const int st_kind = wave;
  // Running source pointers of the prefetch cursor, advanced by wave-uniform steps: no 64-bit
  // multiplies inside the loop.  A step goes to the next head of the same query tile, a wrap from
  // the last head back to the first head of the tile before (dir < 0) or after it.
  const __bf16* q_src = (const __bf16*)a.q + b * a.qs.b + (int64_t)(hk * G) * a.qs.h + (int64_t)t_first * Tile::BQ * a.qs.s;
  const __bf16* d_src = (const __bf16*)a.dout + b * a.dos.b + (int64_t)(hk * G) * a.dos.h + (int64_t)t_first * Tile::BQ * a.dos.s;
  const int64_t stat_row0 = ((int64_t)b * a.stat_hq + hk * G) * a.T + (int64_t)t_first * Tile::BQ;
  const bool s_is_seg = HAS_SEG && st_kind == 2;
  const char* s_src = st_kind == 1 ? (const char*)(a.ndelta + stat_row0) : (const char*)(a.lse2 + stat_row0);  // wave-uniform
  if (s_is_seg) s_src = (const char*)(a.seg + (int64_t)b * a.T + (int64_t)t_first * Tile::BQ);
  const unsigned s_lane = 16 * (lane & 7);  // lanes 0..7 fetch 4 query rows each
  const int64_t q_step = a.qs.h, d_step = a.dos.h;
  const int64_t q_wrap = -(int64_t)(G - 1) * a.qs.h + dir * (int64_t)Tile::BQ * a.qs.s;
  const int64_t d_wrap = -(int64_t)(G - 1) * a.dos.h + dir * (int64_t)Tile::BQ * a.dos.s;
  // statistics rows are [B, Hq, T] fp32; segment ids do not depend on the head
  const int64_t s_step = s_is_seg ? 0 : (int64_t)a.T * 4;
  const int64_t s_wrap = s_is_seg ? dir * (int64_t)Tile::BQ * 4 : (-(int64_t)(G - 1) * a.T + dir * Tile::BQ) * 4;
  const unsigned lds0 = lds_address(smem);
  // The k-th group of loads (Q rows, dO rows, statistics) of the cursor's tile into the buffer at LDS
  // address BUF_; all from scalar bases, no vector instruction forms an address.
  constexpr int NGRP = 3;
#define AXL_DMA(BUF_, K_)                                                                          \
  {                                                                                               \
    if ((K_) == 0) {                                                                              \
      if constexpr (PAIRS) dma16x2(q_lane[0], q_lane[Tile::DMA_PER_WAVE - 1], q_src, (BUF_) + wave * (8 * Tile::ROWB)); \
      else dma16s(q_lane[0], q_src, (BUF_) + wave * (8 * Tile::ROWB));                            \
    } else if ((K_) == 1) {                                                                       \
      if constexpr (PAIRS) dma16x2(d_lane[0], d_lane[Tile::DMA_PER_WAVE - 1], d_src, (BUF_) + Tile::TILE_BYTES + wave * (8 * Tile::ROWB)); \
      else dma16s(d_lane[0], d_src, (BUF_) + Tile::TILE_BYTES + wave * (8 * Tile::ROWB));         \
    } else {                                                                                      \
      dma16s_first8(s_lane, s_src, (BUF_) + Tile::STAT_BASE + st_kind * (Tile::BQ * 4));          \
    }                                                                                             \
  }
#define AXL_DMA_TILE(BUF_)                                                                         \
  {                                                                                               \
    AXL_DMA(BUF_, 0) AXL_DMA(BUF_, 1) AXL_DMA(BUF_, 2)                                            \
  }
  // Prefetch cursor; it stops at the last tile (re-fetching that tile is harmless).
  int pf_idx = 0, pf_t = t_first - t_begin, pf_h = 0;  // tile number, query tile (from t_begin), head within the group
#define AXL_ADVANCE()                                                       \
  {                                                                         \
    const bool adv_ = pf_idx + 1 < total;                                   \
    const bool wrap_ = adv_ && (pf_h + 1 == G);                             \
    pf_idx += adv_ ? 1 : 0;                                                 \
    pf_h = wrap_ ? 0 : pf_h + (adv_ ? 1 : 0);                               \
    pf_t += wrap_ ? dir : 0;                                                \
    q_src += adv_ ? (wrap_ ? q_wrap : q_step) : 0;                          \
    d_src += adv_ ? (wrap_ ? d_wrap : d_step) : 0;                          \
    s_src += adv_ ? (wrap_ ? s_wrap : s_step) : 0;                          \
  }

  char* buf_b = smem;                         // tile j     (stage B reads)
  char* buf_e = smem + Tile::BUF_BYTES;       // tile j + 1 (next stage B; its statistics are in registers)
  char* buf_a = smem + 2 * Tile::BUF_BYTES;   // tile j + 2 (stage A reads)
  char* buf_n = smem + 3 * Tile::BUF_BYTES;   // tile j + 3 (requested two iterations ago, awaited at the end of this one)
  char* buf_s = smem + 4 * Tile::BUF_BYTES;   // tile j + 4 (requested one iteration ago)
  char* buf_s2 = smem + 5 * Tile::BUF_BYTES;  // tile j + 5 (requested during this iteration)

  // Per-lane read offsets (bytes) into a swizzled tile.  Stage A: row swap_bits_2_3(l32), logical
  // chunk 2kk + g.  Stage B (transposing reads): row 8g + j16/4 (+4 for the second half, +16 for the
  // second group of 16 queries), logical byte column (16 half + 4 (j16 % 4)) * 2 + 64 dt.
  const int a_row = swap_bits_2_3(l32);
  const int a_row_off = a_row * Tile::ROWB;
  const int a_xor = tile_swizzle<D>(a_row) << 4;
  const int j16 = lane & 15, half = (lane >> 4) & 1;
  const int t_row = 8 * g + (j16 >> 2);
  const int t_col = (16 * half + 4 * (j16 & 3)) * 2;
  const int t_off0 = t_row * Tile::ROWB + (t_col & 15), t_off1 = t_off0 + 4 * Tile::ROWB;
  const int t_xor0 = tile_swizzle<D>(t_row) << 4, t_xor1 = tile_swizzle<D>(t_row + 4) << 4;
#define AXL_A_FRAG(BUF_, WHICH_, KK_) \
  (*(const bf16x8*)((BUF_) + (WHICH_) * Tile::TILE_BYTES + a_row_off + ((((KK_) * 32) + g * 16) ^ a_xor)))

  // Three tiles are in flight: stage A (S = Q K^T, dP = dO V^T) of tile j+2, the elementwise stage
  // (P = exp2(S c - lse), dS = P (dP - delta)) of tile j+1 and stage B (dV^T += dO^T P,
  // dK^T += Q^T dS) of tile j; tile j+3 is landing in LDS and tile j+4 is requested.  Everything
  // that is not an MFMA - elementwise arithmetic, operand packing, LDS fragment reads, tile load
  // requests, pointer updates - is dealt out over the MFMA slots of the iteration, so the matrix
  // pipe never waits for it.
  // Two register sets that swap roles from iteration to iteration, so nothing is copied: in an
  // iteration one holds tile j + 1 (logits / dP, turned into P / dS) and tile j's packed operands,
  // the other receives the stage-A accumulators of tile j + 2 and tile j + 1's packed operands.
  // (s_e, dp_e, pb, dsb) is the first kind on entry to every run of iterations.
  floatx16 s_e, dp_e, s_x, dp_x;
  union PackedOperand {
    bf16x8 v[2];
    bf16x2 p[8];
  };
  PackedOperand pb, dsb, pb_x, dsb_x;
#pragma unroll
  for (int r = 0; r < 16; r++) s_e[r] = dp_e[r] = 0.f;

  floatx4 lse_v[4], del_v[4];
  intx4 seg_v[4];
  int diff0 = 0;
  // Row statistics of the tile in BUF_: register r of lane group g is query q0 + 16(r/8) + 8g + (r%8).
#define AXL_READ_STATS_PART(BUF_, T8_, LSE_, DEL_, SEG_)                                \
  {                                                                                     \
    const char* st_ = (BUF_) + Tile::STAT_BASE + 8 * g * 4;                             \
    LSE_[2 * (T8_)] = *(const floatx4*)(st_ + 64 * (T8_));                              \
    LSE_[2 * (T8_) + 1] = *(const floatx4*)(st_ + 64 * (T8_) + 16);                     \
    DEL_[2 * (T8_)] = *(const floatx4*)(st_ + Tile::BQ * 4 + 64 * (T8_));               \
    DEL_[2 * (T8_) + 1] = *(const floatx4*)(st_ + Tile::BQ * 4 + 64 * (T8_) + 16);      \
    if (HAS_SEG) {                                                                      \
      SEG_[2 * (T8_)] = *(const intx4*)(st_ + 2 * Tile::BQ * 4 + 64 * (T8_));           \
      SEG_[2 * (T8_) + 1] = *(const intx4*)(st_ + 2 * Tile::BQ * 4 + 64 * (T8_) + 16);  \
    }                                                                                   \
  }
  // Elementwise stage of element R_ of (s_e, dp_e) in three phases which the pipelined loop issues in
  // three consecutive MFMA slots, so that no instruction waits for the result of the one before it
  // (v_exp_f32 in particular has a long latency): exponent, exponential, products.  MASKED_ selects
  // the mask arithmetic (tiles that no mask touches run without it).
#define AXL_ELEM_1(R_, MASKED_)                                                                \
  {                                                                                            \
    const int r_ = (R_);                                                                       \
    float sv_ = s_e[r_];                                                                       \
    if (MASKED_) {                                                                             \
      const unsigned diff_ = (unsigned)(diff0 + 16 * (r_ / 8) + (r_ % 8));                     \
      sv_ = diff_ <= limit ? sv_ : kMasked;                                                    \
      if (HAS_SEG) sv_ = seg_v[r_ / 4][r_ % 4] == seg_k ? sv_ : kMasked;                       \
    }                                                                                          \
    float off_ = lse_v[r_ / 4][r_ % 4]; /* -lse * log2 e */                                    \
    if constexpr (HAS_BIAS) {                                                                  \
      /* bias raw bits: fp32 as loaded, bf16 in the low half.  The empty statement keeps the    \
         first use of the loaded register here, an iteration after its load: without it the     \
         shift (and the test of the dropout byte below) moves up to the load and waits there    \
         for everything in flight. */                                                           \
      uint32_t bw_ = braw_v[r_];                                                               \
      asm volatile("" : "+v"(bw_));                                                            \
      off_ = __builtin_fmaf(__builtin_bit_cast(float, bw_ << (BIAS_F32 ? 0 : 16)), kLog2e, off_); \
    }                                                                                          \
    s_e[r_] = __builtin_fmaf(sv_, c, off_);                                                    \
  }
#define AXL_ELEM_2(R_) s_e[R_] = fast_exp2(s_e[R_]);
#define AXL_ELEM_3(R_)                                                                         \
  {                                                                                            \
    const int r_ = (R_);                                                                       \
    const float p_ = s_e[r_];                                                                  \
    float dpv_ = dp_e[r_];                                                                     \
    if constexpr (HAS_DROP) {                                                                  \
      uint32_t dw_ = draw_v[r_];                                                               \
      asm volatile("" : "+v"(dw_));                                                            \
      const bool kept_ = dw_ == 0;                                                             \
      dpv_ = kept_ ? dpv_ * a.aux.keep_scale : 0.f; /* gpu_attention.py:509-512 */            \
      s_e[r_] = kept_ ? p_ : 0.f; /* P that multiplies dO: dropped entries removed */          \
    }                                                                                          \
    if constexpr (AUX) dp_e[r_] = p_ * (dpv_ + del_v[r_ / 4][r_ % 4]); /* del_v holds -delta */ \
    else dp_e[r_] = p_ * dpv_; /* the dP chain started from -delta */                          \
  }
#define AXL_ELEM(R_)                                                                           \
  {                                                                                            \
    AXL_ELEM_1(R_, true)                                                                       \
    AXL_ELEM_2(R_)                                                                             \
    AXL_ELEM_3(R_)                                                                             \
  }
  // Dense bias / dropout mask (AUX): this lane's key column of the 16 query rows of a tile, one
  // element per register, requested a whole iteration before the elementwise stage consumes it.  Two
  // register sets swap roles from iteration to iteration (a copy would have to wait for the loads).
  // Which inputs there are and the bias element type are template arguments, so the requests are
  // straight-line code and the compiler's wait counts for them stay exact.
  uint32_t braw_v[16], draw_v[16], braw_w[16], draw_w[16];
#pragma unroll
  for (int r = 0; r < 16; r++) braw_v[r] = draw_v[r] = braw_w[r] = draw_w[r] = 0;
  constexpr int bias_es = BIAS_F32 ? 4 : 2;
#define AXL_AUX_ROW0(H_, Q0_, BP_, DP_)                                                              \
  {                                                                                                  \
    const int64_t head_ = hk * G + (H_), row_ = (Q0_) + 8 * g;                                       \
    BP_ = HAS_BIAS ? a.aux.bias + b * a.aux.bias_sb + head_ * a.aux.bias_sh + row_ * a.aux.bias_sr + \
                         (int64_t)kpos * bias_es                                                     \
                   : nullptr;                                                                        \
    DP_ = HAS_DROP ? a.aux.drop + b * a.aux.drop_sb + head_ * a.aux.drop_sh + row_ * a.aux.drop_sr + kpos \
                   : nullptr;                                                                        \
  }
#define AXL_AUX_LOAD(BP_, DP_, R_, BDST_, DDST_)                                                     \
  {                                                                                                  \
    const int64_t rr_ = 16 * ((R_) / 8) + ((R_) % 8);                                                \
    if constexpr (HAS_BIAS) {                                                                        \
      const char* e_ = (BP_) + rr_ * a.aux.bias_sr;                                                  \
      if constexpr (BIAS_F32) BDST_[R_] = *(const uint32_t*)e_;                                      \
      else BDST_[R_] = *(const uint16_t*)e_;                                                         \
    }                                                                                                \
    if constexpr (HAS_DROP) DDST_[R_] = *((DP_) + rr_ * a.aux.drop_sr);                              \
  }
#define AXL_PACK_PAIR(PB_, DSB_, I_)                                    \
  {                                                                     \
    PB_.p[I_] = E::pack(s_e[2 * (I_)], s_e[2 * (I_) + 1]);            \
    DSB_.p[I_] = E::pack(dp_e[2 * (I_)], dp_e[2 * (I_) + 1]);         \
  }
  // Ahead of the inline-assembly chains of a pipeline-fill tile, whose accumulators vector ALU
  // instructions have just set (zeros, -delta): a matrix instruction that reads, as its addend, a
  // register which a vector ALU instruction wrote right before it gets a stale value, and the
  // compiler, which keeps that distance for its own MFMAs, does not know what the assembly is.  The
  // wait below is placed after whatever wrote the registers and before the first MFMA.
#define AXL_CHAIN_START(S_, DP_) \
  if constexpr (!AUX) asm volatile("s_nop 7" : "+v"(S_), "+v"(DP_));
  // Stage A of the tile in BUF_ into (S_, DP_), not interleaved with anything (pipeline fill).
#define AXL_STAGE_A_PLAIN(BUF_, S_, DP_)                                                        \
  _Pragma("unroll") for (int kk = 0; kk < KK; kk++) {                                           \
    const bf16x8 qa_ = AXL_A_FRAG(BUF_, 0, kk);                                                 \
    const bf16x8 da_ = AXL_A_FRAG(BUF_, 1, kk);                                                 \
    if constexpr (AUX) {                                                                        \
      S_ = E::mfma_32x32x16(qa_, kf[kk], S_);                                                   \
      DP_ = E::mfma_32x32x16(da_, vf[kk], DP_);                                                 \
    } else if (kk + 1 < KK) {                                                                   \
      E::mfma_32x32x16_vgpr(qa_, kf[kk], S_);                                                   \
      E::mfma_32x32x16_vgpr(da_, vf[kk], DP_);                                                  \
    } else {                                                                                    \
      E::mfma_32x32x16_vgpr_last(qa_, kf[kk], S_);                                              \
      E::mfma_32x32x16_vgpr_last(da_, vf[kk], DP_);                                             \
    }                                                                                           \
  }
  union TrFrag {
    bf16x8 v;
    shortx4 hlf[2];
  };
#define AXL_B_READ_FROM(BUF_, DST_, N_)                                                          \
  {                                                                                              \
    const char* p_ = (BUF_) + (((N_) % 2) == 0 ? Tile::TILE_BYTES : 0) + 16 * ((N_) / (2 * DT)) * Tile::ROWB; \
    const int col_ = (t_col & ~15) + (((N_) % (2 * DT)) / 2) * 64;                               \
    DST_.hlf[0] = lds_read_tr16(p_ + t_off0 + (col_ ^ t_xor0));                                  \
    DST_.hlf[1] = lds_read_tr16(p_ + t_off1 + (col_ ^ t_xor1));                                  \
  }

  // The same reads inside the loop, from per-lane offsets that are computed once: per iteration only
  // the ring buffer's base is added (the Q / dO tile and the 16-row group are immediate offsets).
  int a_off[KK], tb_off[2][DT];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) a_off[kk] = a_row_off + ((kk * 32 + g * 16) ^ a_xor);
#pragma unroll
  for (int dt = 0; dt < DT; dt++) {
    tb_off[0][dt] = t_off0 + (((t_col & ~15) + dt * 64) ^ t_xor0);
    tb_off[1][dt] = t_off1 + (((t_col & ~15) + dt * 64) ^ t_xor1);
  }
#define AXL_B_READ_AT(AD_, DST_, N_)                                                             \
  {                                                                                              \
    const int imm_ = (((N_) % 2) == 0 ? Tile::TILE_BYTES : 0) + 16 * ((N_) / (2 * DT)) * Tile::ROWB;     \
    DST_.hlf[0] = lds_read_tr16(AD_[0][((N_) % (2 * DT)) / 2] + imm_);                           \
    DST_.hlf[1] = lds_read_tr16(AD_[1][((N_) % (2 * DT)) / 2] + imm_);                           \
  }

  constexpr int NS = NA + NB;          // MFMAs per iteration: stage B of tile j, then stage A of tile j+2
  constexpr int ESTEP = NS / 16;       // bias / dropout loads: one of the 16 elements per lane every ESTEP slots
  static_assert(NS % 16 == 0, "the 16 elements per lane are spread evenly over the MFMA slots");
  constexpr int kAheadA = 6, kAheadB = 4;
  constexpr int NLD = Tile::DMA_PER_TILE;     // direct-to-LDS loads of a tile per wavefront
  constexpr int LD_SLOT0 = 2;                 // one per slot from here on, after the cursor moved in slot 1
  static_assert(LD_SLOT0 + NLD <= NS, "the loads of a tile fit into one iteration");
  TrFrag bfr_next[kAheadB];            // first stage-B fragments of the next iteration
  int q0_a = t_first * Tile::BQ, q0_s = q0_a, q0_s2 = q0_a;  // first query of tiles j+2, j+3 and j+4
  int h_a = 0, h_s = 0, h_s2 = 0;                            // and their heads within the group

  if (total > 0) {
    // Everything the compiler tracks (stationary fragments, segment ids) has landed before the first
    // untracked load, so its own wait counts never cover a tile load.
    wait_all_vmem();
    AXL_DMA_TILE(lds_address(buf_b))
    AXL_ADVANCE()
    const int q0_1 = (t_begin + pf_t) * Tile::BQ, h_1 = pf_h;
    AXL_DMA_TILE(lds_address(buf_e))
    AXL_ADVANCE()
    q0_a = (t_begin + pf_t) * Tile::BQ;
    h_a = pf_h;
    AXL_DMA_TILE(lds_address(buf_a))
    AXL_ADVANCE()
    q0_s = (t_begin + pf_t) * Tile::BQ;
    h_s = pf_h;
    AXL_DMA_TILE(lds_address(buf_n))
    AXL_ADVANCE()
    q0_s2 = (t_begin + pf_t) * Tile::BQ;
    h_s2 = pf_h;
    AXL_DMA_TILE(lds_address(buf_s))
    if constexpr (AUX) {                 // bias / dropout columns of tile 0
      const char* bp_;
      const uint8_t* dp_;
      AXL_AUX_ROW0(0, t_first * Tile::BQ, bp_, dp_)
#pragma unroll
      for (int r = 0; r < 16; r++) AXL_AUX_LOAD(bp_, dp_, r, braw_v, draw_v)
    }
    wait_all_vmem();  // tiles 0..3 have landed; nothing issued before the loop is pending
    __syncthreads();
    // Pipeline fill: stage A and the elementwise stage of tile 0, stage A of tile 1.
    AXL_READ_STATS_PART(buf_b, 0, lse_v, del_v, seg_v)
    AXL_READ_STATS_PART(buf_b, 1, lse_v, del_v, seg_v)
    if constexpr (!AUX) {  // the dP chain starts from -delta
#pragma unroll
      for (int r = 0; r < 16; r++) dp_e[r] = del_v[r / 4][r % 4];
    }
    AXL_CHAIN_START(s_e, dp_e)
    AXL_STAGE_A_PLAIN(buf_b, s_e, dp_e)
    diff0 = (t_first * Tile::BQ + a.q_off + 8 * g) - kpos;
#pragma unroll
    for (int r = 0; r < 16; r++) AXL_ELEM(r)
#pragma unroll
    for (int i = 0; i < 8; i++) AXL_PACK_PAIR(pb, dsb, i)
#pragma unroll
    for (int r = 0; r < 16; r++) s_e[r] = dp_e[r] = 0.f;
    AXL_READ_STATS_PART(buf_e, 0, lse_v, del_v, seg_v)
    AXL_READ_STATS_PART(buf_e, 1, lse_v, del_v, seg_v)
    if constexpr (!AUX) {
#pragma unroll
      for (int r = 0; r < 16; r++) dp_e[r] = del_v[r / 4][r % 4];
    }
    AXL_CHAIN_START(s_e, dp_e)
    AXL_STAGE_A_PLAIN(buf_e, s_e, dp_e)
    if constexpr (AUX) {                 // ... and of tile 1, for the first iteration
      const char* bp_;
      const uint8_t* dp_;
      AXL_AUX_ROW0(h_1, q0_1, bp_, dp_)
#pragma unroll
      for (int r = 0; r < 16; r++) AXL_AUX_LOAD(bp_, dp_, r, braw_v, draw_v)
    }
    diff0 = (q0_1 + a.q_off + 8 * g) - kpos;  // query of r == 0 minus this lane's key
#pragma unroll
    for (int i = 0; i < kAheadB; i++) AXL_B_READ_FROM(buf_b, bfr_next[i], i)
  }
  // On every path into the loops below, including the one around the block above, nothing the
  // compiler tracks is pending any more.  Without this its wait-count pass carries the loads of the
  // stationary K / V fragments into the loop and covers each fragment's first use there with a
  // vmcnt wait, down to vmcnt(0): every iteration would then wait for the tile loads it has just
  // issued, which the pass cannot see and which are meant to stay in flight for two more iterations.
  wait_all_vmem();

  const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // Iterations [j_from, j_to); MASKED_C says whether their elementwise tiles (j + 1) need mask
  // arithmetic.  The loop is instantiated once per run of iterations of one kind instead of branching
  // inside one loop.
  auto run = [&](int j_from, int j_to, auto masked_c) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_c)::value;
  // One iteration.  (s_e, dp_e): tile j + 1; (pb, dsb): tile j, packed; (s_a, dp_a): the stage-A
  // accumulators of tile j + 2; (pb_n, dsb_n): tile j + 1, packed as its elements complete.
  // Without a bias / dropout mask the stage-A chains accumulate in vector registers
  // (mfma_32x32x16_vgpr): the next iteration's elementwise stage reads them where they are.  Its first
  // read of s comes after that iteration's first MFMA and after the last MFMA of the dP chain, its
  // first read of dp two slots later.  The bias / dropout instantiations, which run out of vector
  // registers, keep the compiler's own form.
  auto iter = [&](floatx16& s_e, floatx16& dp_e, PackedOperand& pb, PackedOperand& dsb, floatx16& s_a, floatx16& dp_a,
                  PackedOperand& pb_n, PackedOperand& dsb_n, uint32_t (&braw_v)[16], uint32_t (&draw_v)[16],
                  uint32_t (&braw_n)[16], uint32_t (&draw_n)[16]) __attribute__((always_inline)) {
    bf16x8 afr[NA];
    TrFrag bfr[NB];
#pragma unroll
    for (int i = 0; i < kAheadB; i++) bfr[i] = bfr_next[i];
    int q0_p = q0_s2, h_p = h_s2;
    const unsigned lds_s = lds_address(buf_s2);
    const char* a_ad[KK];                // this iteration's fragment addresses: stage A in tile j+2,
    const char* b_ad[2][DT];             // stage B in tile j,
    const char* e_ad[2][DT];             // and the first stage-B fragments of tile j+1
#pragma unroll
    for (int kk = 0; kk < KK; kk++) a_ad[kk] = buf_a + a_off[kk];
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      b_ad[0][dt] = buf_b + tb_off[0][dt];
      b_ad[1][dt] = buf_b + tb_off[1][dt];
      e_ad[0][dt] = buf_e + tb_off[0][dt];
      e_ad[1][dt] = buf_e + tb_off[1][dt];
    }
    const char* bias_t = nullptr;        // bias / dropout columns of tile j + 2 go to (braw_n, draw_n)
    const uint8_t* drop_t = nullptr;
    if constexpr (AUX) AXL_AUX_ROW0(h_a, q0_a, bias_t, drop_t)
    if constexpr (SPILL) {
      // dS of tile j (this iteration's stage-B operand), ahead of the iteration's tile loads: by the
      // end of the iteration the stores have long been accepted.
      store16x2(ds_lane, ds_ptr, dsb.v[0], dsb.v[1]);
      // next head of the same tile (one run further), or head 0 of the tile before (G runs of that
      // tile back from head 0 of this one) or of the tile after (which is the next run as well)
      const bool wrap_ = st_h + 1 == G;
      const int run_ = 4 * ((st_t >> 2) + 1) * kDsBlockBytes, run_prev_ = 4 * (((st_t - 1) >> 2) + 1) * kDsBlockBytes;
      ds_ptr += wrap_ && dir < 0 ? -(int64_t)((G - 1) * run_ + G * run_prev_) : (int64_t)run_;
      st_h = wrap_ ? 0 : st_h + 1;
      st_t += wrap_ ? dir : 0;
    }
    __builtin_amdgcn_sched_barrier(0);
    // One MFMA slot.  The slot number is a compile-time constant (the slots are instantiated one by
    // one, not produced by a loop unroller, which gives up on bodies of this size).
    auto slot = [&](auto n_c) __attribute__((always_inline)) {
      constexpr int n = decltype(n_c)::value;
      // ---- LDS fragments requested ahead of their MFMA
      if constexpr (n + kAheadB < NB) AXL_B_READ_AT(b_ad, bfr[n + kAheadB], n + kAheadB)
      if constexpr (n + kAheadA >= NB && n + kAheadA - NB < NA) {
        constexpr int x = n + kAheadA - NB;
        afr[x] = *(const bf16x8*)(a_ad[x / 2] + (x % 2) * Tile::TILE_BYTES);
      }
      if constexpr (n >= NS - kAheadB) AXL_B_READ_AT(e_ad, bfr_next[n - (NS - kAheadB)], n - (NS - kAheadB))
      // ---- the MFMA of this slot.  Stage-B step m = t8 * 2DT + dt * 2 + which (which 0: dV with the
      // dO^T fragment and P, 1: dK with the Q^T fragment and dS); stage-A step x: even -> S chain
      // with Q fragment x/2, odd -> dP chain with dO fragment x/2.
      if constexpr (n < NB) {
        constexpr int t8 = n / (2 * DT), dt = (n % (2 * DT)) / 2;
        if constexpr (n % 2 == 0)
          dv_acc[dt] = E::mfma_32x32x16(bfr[n].v, pb.v[t8], dv_acc[dt]);
        else
          dk_acc[dt] = E::mfma_32x32x16(bfr[n].v, dsb.v[t8], dk_acc[dt]);
      } else {
        constexpr int x = n - NB;
        if constexpr (AUX) {
          if constexpr (x % 2 == 0) s_a = E::mfma_32x32x16(afr[x], kf[x / 2], x == 0 ? zero16 : s_a);
          else dp_a = E::mfma_32x32x16(afr[x], vf[x / 2], x == 1 ? zero16 : dp_a);
        } else {
          if constexpr (x == 0) E::mfma_32x32x16_vgpr_zero(afr[x], kf[x / 2], s_a);
          else if constexpr (x % 2 == 0) E::mfma_32x32x16_vgpr(afr[x], kf[x / 2], s_a);
          else E::mfma_32x32x16_vgpr(afr[x], vf[x / 2], dp_a);  // the chain starts from -delta
        }
      }
      // The first elementwise read of (s_e, dp_e) stays behind this slot's MFMA: two MFMAs then lie
      // between it and the last MFMA of the S chain, whatever the barrier in between took.
      if constexpr (n == 0) __builtin_amdgcn_sched_barrier(0);
      // ---- elementwise stage of tile j+1: element e starts in slot e (NS-3)/16 and takes three
      // slots; pairs are packed one slot after their second element is complete
#pragma unroll
      for (int e = 0; e < 16; e++) {
        if (e * (NS - 3) / 16 + 2 == n) AXL_ELEM_3(e)
        if (e * (NS - 3) / 16 + 1 == n) AXL_ELEM_2(e)
        if (e * (NS - 3) / 16 == n) AXL_ELEM_1(e, MASKED)
      }
#pragma unroll
      for (int i = 0; i < 8; i++)
        if ((2 * i + 1) * (NS - 3) / 16 + 3 == n) AXL_PACK_PAIR(pb_n, dsb_n, i)
      // ---- tile j+4: advance the cursor, then one direct-to-LDS load per slot
      if (n == LD_SLOT0 - 1) {
        AXL_ADVANCE()
        q0_p = (t_begin + pf_t) * Tile::BQ;
        h_p = pf_h;
      }
      if constexpr (AUX) {
        if (n % ESTEP == 0) AXL_AUX_LOAD(bias_t, drop_t, n / ESTEP, braw_n, draw_n)
      }
      if constexpr (n >= LD_SLOT0 && n < LD_SLOT0 + NGRP) AXL_DMA(lds_s, n - LD_SLOT0)
      // ---- statistics of tile j+2 for the next iteration's elementwise stage, four query rows at a
      // time, each group as soon as this iteration's elements are done with the registers
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const char* st_ = buf_a + Tile::STAT_BASE + 8 * g * 4 + 64 * (i / 2) + 16 * (i % 2);
        if (n == (4 * i + 3) * (NS - 3) / 16 + 1) {
          lse_v[i] = *(const floatx4*)st_;
          if (HAS_SEG) seg_v[i] = *(const intx4*)(st_ + 2 * Tile::BQ * 4);
        }
        if constexpr (AUX) {
          if (n == (4 * i + 3) * (NS - 3) / 16 + 3) del_v[i] = *(const floatx4*)(st_ + Tile::BQ * 4);
        } else {
          // -delta of tile j+2's rows: what its dP chain starts from (slot NB + 1), loaded into the
          // accumulator itself (the register set is idle until then)
          if (n == NB - 4 + i) {
            const floatx4 d4 = *(const floatx4*)(st_ + Tile::BQ * 4);
            dp_a[4 * i] = d4[0]; dp_a[4 * i + 1] = d4[1]; dp_a[4 * i + 2] = d4[2]; dp_a[4 * i + 3] = d4[3];
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    for_each_index<NS>(slot);
    // Tile j+3 (requested two iterations ago) has landed once at most the loads of the last two
    // iterations are outstanding (loads complete in issue order; the dS stores of the spill path may
    // complete out of order with them, which only makes the count stricter); after the barrier every
    // wavefront's part of it is visible, and nobody reads tile j's buffer any more, which the next
    // iteration refills.  (With a bias or a dropout mask, at least 43 of their element loads - 11 of
    // the iteration before last, 16 of each iteration since - are younger than tile j+3's loads as
    // well; 40 leaves a margin.)
    wait_vmem_le<2 * NLD + (AUX ? 40 : 0)>();
    __syncthreads();
    // The stage-A chains of the last slots were issued through inline assembly, so the compiler places
    // no wait states behind them; where a run of iterations ends it may move values into their
    // registers a few instructions after this barrier.  Eight wait states here bring every such write
    // to at least the 12 the hardware wants after the last MFMA of a chain, whatever the barrier took.
    if constexpr (!AUX) asm volatile("s_nop 7");
    char* const tmp = buf_b;
    buf_b = buf_e;
    buf_e = buf_a;
    buf_a = buf_n;
    buf_n = buf_s;
    buf_s = buf_s2;
    buf_s2 = tmp;
    diff0 = (q0_a + a.q_off + 8 * g) - kpos;
    q0_a = q0_s;
    q0_s = q0_s2;
    q0_s2 = q0_p;
    h_a = h_s;
    h_s = h_s2;
    h_s2 = h_p;
  };
    int j = j_from;
    for (; j + 1 < j_to; j += 2) {
      iter(s_e, dp_e, pb, dsb, s_x, dp_x, pb_x, dsb_x, braw_v, draw_v, braw_w, draw_w);
      iter(s_x, dp_x, pb_x, dsb_x, s_e, dp_e, pb, dsb, braw_w, draw_w, braw_v, draw_v);
    }
    if (j < j_to) {
      // odd count: one more iteration, then the sets go back to their roles with one copy per run
      iter(s_e, dp_e, pb, dsb, s_x, dp_x, pb_x, dsb_x, braw_v, draw_v, braw_w, draw_w);
      if constexpr (!AUX) asm volatile("s_nop 15\n\ts_nop 3" : "+v"(s_x), "+v"(dp_x));  // the chains have just ended
      s_e = s_x;
      dp_e = dp_x;
      pb = pb_x;
      dsb = dsb_x;
      if constexpr (AUX) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          braw_v[r] = braw_w[r];
          draw_v[r] = draw_w[r];
        }
      }
    }
  };
  // Query tile t (counted from t_begin) needs no mask for this wavefront's 32 keys when its queries
  // all see them: t in [u_lo, u_hi].  In processing order tile number e is query tile nt - 1 - e / G
  // (walking down) or e / G (walking up) of head e % G, and the elementwise tile of iteration j is
  // e = j + 1.
  auto floor_div = [](int x, int y) { return x >= 0 ? x / y : -((-x + y - 1) / y); };
  int u_lo = 0, u_hi = nt - 1;
  if (a.mask_kind != AXL_MASK_NONE) {
    u_lo = max(0, floor_div(k0 + 31 - a.q_off + Tile::BQ - 1, Tile::BQ) - t_begin);
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW)
      u_hi = min(nt - 1, floor_div(a.window + k0 - 31 - a.q_off, Tile::BQ) - t_begin);
  }
  if (HAS_SEG && !AUX) {
    // Query tiles whose 32 rows all carry the segment id that all 32 keys of this wavefront carry
    // need no segment mask either: take the first run [tA, tB) of such tiles (the masked loop is
    // always correct, so whatever lies outside that run simply stays on it).
    int tA = 0, tB = 0;
    const int sub0 = t_begin - sub_g0;   // table index of query tile t_begin
    if (sub0 + nt <= kMaxSubDkv) {
      const int wk_id = __builtin_amdgcn_readfirstlane(seg_k);
      const bool k_uniform = __builtin_amdgcn_ballot_w64(seg_k != wk_id) == 0 && wk_id != kNotUniformDkv;
      tA = tB = nt;
      if (k_uniform) {
        for (int base = 0; base < nt && tA == nt; base += 64) {
          const int i = base + lane;
          const uint64_t m = __builtin_amdgcn_ballot_w64(i < nt && s_sub[sub0 + min(i, nt - 1)] == wk_id);
          if (m) tA = base + __builtin_ctzll(m);
        }
        for (int base = tA & ~63; base < nt && tB == nt; base += 64) {
          const int i = base + lane;
          const uint64_t m = __builtin_amdgcn_ballot_w64(i > tA && i < nt && s_sub[sub0 + min(i, nt - 1)] != wk_id);
          if (m) tB = base + __builtin_ctzll(m);
        }
      }
    }
    u_lo = max(u_lo, tA);
    u_hi = min(u_hi, tB - 1);
  }
  u_lo = min(u_lo, nt);
  u_hi = max(u_hi, u_lo - 1);
  if constexpr (AUX) {
    run(0, total, std::true_type{});  // every tile takes the masked path
  } else {
    int j = 0;
    auto run_to = [&](int e_end, auto masked_c) __attribute__((always_inline)) {
      const int j_end = min(total, e_end - 1);
      run(j, j_end, masked_c);
      j = max(j, j_end);
    };
    // walking down: far end of a sliding window, interior, down to the diagonal; walking up: the reverse
    run_to(dir < 0 ? G * (nt - 1 - u_hi) : G * u_lo, std::true_type{});
    run_to(dir < 0 ? G * (nt - u_lo) : G * (u_hi + 1), std::false_type{});
    run_to(total, std::true_type{});
    run(j, total, std::true_type{});  // the last iteration (its elementwise tile is past the end)
  }
#undef AXL_AUX_ROW0
#undef AXL_AUX_LOAD
  // The cursor re-requests the last tile during the final iterations (which keeps the count of
  // outstanding loads the same in every iteration); none of those may still be in flight when this
  // workgroup's LDS is handed to the next one.
  wait_all_vmem();
#undef AXL_READ_STATS_PART
#undef AXL_ELEM
#undef AXL_ELEM_1
#undef AXL_ELEM_2
#undef AXL_ELEM_3
#undef AXL_PACK_PAIR
#undef AXL_STAGE_A_PLAIN
#undef AXL_CHAIN_START
#undef AXL_B_READ_FROM
#undef AXL_B_READ_AT
#undef AXL_DMA
#undef AXL_DMA_TILE
#undef AXL_A_FRAG
#undef AXL_ADVANCE

  __bf16* dkp = (__bf16*)a.dk + b * a.dks.b + (int64_t)(k0 + l32) * a.dks.s + hk * a.dks.h;
  __bf16* dvp = (__bf16*)a.dv + b * a.dvs.b + (int64_t)(k0 + l32) * a.dvs.s + hk * a.dvs.h;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int rq = 0; rq < 4; rq++) {
      union {
        bf16x2 p[2];
        uint2 u;
      } w;
      w.p[0] = E::pack(dk_acc[dt][4 * rq + 0] * a.scale, dk_acc[dt][4 * rq + 1] * a.scale);
      w.p[1] = E::pack(dk_acc[dt][4 * rq + 2] * a.scale, dk_acc[dt][4 * rq + 3] * a.scale);
      const bool in_row = 32 * dt + 8 * rq + 4 * g < a.d_real;
      if (in_row) *(uint2*)(dkp + 32 * dt + 8 * rq + 4 * g) = w.u;
      const float vs = AUX ? a.aux.keep_scale : 1.0f;  // kept probabilities are P / (1 - rate)
      w.p[0] = E::pack(dv_acc[dt][4 * rq + 0] * vs, dv_acc[dt][4 * rq + 1] * vs);
      w.p[1] = E::pack(dv_acc[dt][4 * rq + 2] * vs, dv_acc[dt][4 * rq + 3] * vs);
      if (in_row) *(uint2*)(dvp + 32 * dt + 8 * rq + 4 * g) = w.u;
    }
  __syncthreads();  // every wavefront is done with the ring before the next key block's first tiles arrive
  }  // key blocks of this workgroup
}

template <typename E, int D, bool HAS_SEG, int AUX, bool SPILL = false>
static hipError_t launch_one(const BwdArgs& a, hipStream_t stream) {
  using Tile = DkvTile<D>;
  auto kernel = flash_bwd_dkdv_kernel<E, D, HAS_SEG, AUX, SPILL>;
  hipError_t err = allow_dynamic_lds((const void*)kernel, Tile::LDS_BYTES);
  if (err != hipSuccess) return err;
  const int grid = (a.S / Tile::BKV) * a.B * a.Hkv / a.kb_per_wg;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), Tile::LDS_BYTES, stream, a);
  return hipGetLastError();
}

template <typename E, int D, int AUX>
static hipError_t launch_seg(const BwdArgs& a, hipStream_t stream) {
  return a.seg ? launch_one<E, D, true, AUX>(a, stream) : launch_one<E, D, false, AUX>(a, stream);
}

template <typename E, int D>
static hipError_t launch_aux(const BwdArgs& a, hipStream_t stream) {
  const int bias = a.aux.bias ? (a.aux.bias_f32 ? kAuxBias32 : kAuxBias16) : 0;
  const int mode = bias | (a.aux.drop ? kAuxDrop : 0);
  switch (mode) {
    case kAuxBias16: return launch_seg<E, D, kAuxBias16>(a, stream);
    case kAuxBias32: return launch_seg<E, D, kAuxBias32>(a, stream);
    case kAuxDrop: return launch_seg<E, D, kAuxDrop>(a, stream);
    case kAuxBias16 | kAuxDrop: return launch_seg<E, D, kAuxBias16 | kAuxDrop>(a, stream);
    default: return launch_seg<E, D, kAuxBias32 | kAuxDrop>(a, stream);
  }
}

template <typename E>
static hipError_t launch_for(const BwdArgs& a, int head_dim, bool aux, hipStream_t stream) {
  const bool seg = a.seg != nullptr;
  if (aux) return head_dim == 128 ? launch_aux<E, 128>(a, stream) : launch_aux<E, 64>(a, stream);
  if (a.ds) {
    if (head_dim == 128)
      return seg ? launch_one<E, 128, true, 0, true>(a, stream) : launch_one<E, 128, false, 0, true>(a, stream);
    return seg ? launch_one<E, 64, true, 0, true>(a, stream) : launch_one<E, 64, false, 0, true>(a, stream);
  }
  return head_dim == 128 ? launch_seg<E, 128, 0>(a, stream) : launch_seg<E, 64, 0>(a, stream);
}

hipError_t launch_bwd_dkdv(const BwdArgs& a, int dtype, int head_dim, bool aux, hipStream_t stream) {
  return dtype == AXL_F16 ? launch_for<ElemF16>(a, head_dim, aux, stream)
                          : launch_for<ElemBf16>(a, head_dim, aux, stream);
}

}  // namespace axl
