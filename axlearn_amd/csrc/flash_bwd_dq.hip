// dQ kernel of the flash-attention backward for gfx950 (bf16).
//
// Replaces axlearn/common/flash_attention/gpu_attention.py:533-616 (`_mha_backward_kernel_dq`):
//   p = exp(qk - lse); dp = dO v^T; ds = p * (dp - delta) * scale; dq += ds k,
// with ds rounded to bf16 before its GEMM and fp32 accumulation (:608).
//
// Mapping.  A workgroup owns 128 query rows of one (batch, query head); each of its 4 wavefronts
// keeps the Q and dO fragments of 32 rows in registers (B operands) together with the fp32 dQ^T
// accumulators of those rows, and loops over the key tiles the rows can see.  Key tiles (64 rows of
// K and V, plus their segment ids) stream through a four-deep LDS ring filled by direct global->LDS
// loads: one unpadded XOR-swizzled copy per tile serves the row-per-lane fragment reads of stage A
// and the transposing reads of stage B without bank conflicts.
//
// One wavefront per SIMD, software pipelined by hand over sub-tiles of 32 keys.  Step j runs
//   stage B of sub-tile j:    dQ^T += K^T dS^T                 (D/16 MFMAs, K^T by transposing LDS reads)
//   stage A of sub-tile j+2:  S^T = K Q^T and dP^T = V dO^T    (2*D/16 MFMAs, lane = query, registers = keys)
//   elementwise of j+1:       P = exp2(S*c - lse), dS = P * (dP - delta), packed to bf16
// and everything that is not an MFMA is dealt out over the MFMA slots of the step.  A loop trip is
// the two steps of one 64-key tile, written out with the roles of the two register sets swapped, so
// no value is copied from "next" to "current".  Trips that no mask touches run a loop without any
// mask arithmetic (the choice is wave-uniform).
#include <type_traits>

#include "flash_bwd.h"

namespace axl {

template <int D, bool HAS_SEG, int NW>
struct DqRing {
  static constexpr int BQ = 32 * NW;         // query rows per workgroup (32 per wavefront)
  static constexpr int BK = 64;              // keys per LDS tile (two sub-tiles of 32)
  static constexpr int ROWB = D * 2;         // bytes per row: unpadded, chunks swizzled (tile_swizzle)
  static constexpr int SUB_BYTES = 32 * ROWB;                    // one sub-tile of K or V
  static constexpr int TILE_BYTES = BK * ROWB;                   // K tile, then the V tile
  static constexpr int SEG_BASE = 2 * TILE_BYTES;
  static constexpr int SEG_BYTES = BK * 4;                       // segment ids of the keys
  static constexpr int BUF_BYTES = SEG_BASE + SEG_BYTES;
  static constexpr int NBUF = 4;
  static constexpr int RPI = 1024 / ROWB;                        // rows per direct-to-LDS instruction
  static constexpr int DMA_PER_WAVE = BK / NW / RPI;             // per tensor per tile (BK / NW rows per wavefront)
  static constexpr int DMA_PER_TILE = 2 * DMA_PER_WAVE + (HAS_SEG ? 1 : 0);
  static constexpr int LDS_BYTES = NBUF * BUF_BYTES;
};

constexpr int kMaxSub = 1024;               // 32-key sub-tiles whose segment ids the dQ kernel classifies
constexpr int kNotUniform = -0x7fffffff - 1;  // marks a sub-tile with more than one segment id

// FUSE_DELTA: the kernel also computes delta = rowsum(out * dO) (gpu_attention.py:653-658) and the
// scaled lse of its own rows and leaves both in the workspace for the dK/dV kernel, which then has to
// run after this one; the separate delta pass is not needed.
template <typename E, int D, bool HAS_SEG, int NW, bool FUSE_DELTA>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(NW / 4, NW / 4)))
void flash_bwd_dq_ring_kernel(const BwdArgs a) {
  using Tile = DqRing<D, HAS_SEG, NW>;
  constexpr int KK = D / 16, DT = D / 32;
  constexpr int NA = 2 * KK;          // stage-A MFMAs per sub-tile
  constexpr int NB = 2 * DT;          // stage-B MFMAs per sub-tile
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  int qb, b, h;
  decode_block(blockIdx.x, (a.T + Tile::BQ - 1) / Tile::BQ, a.B, a.Hq, a.Hkv, 32, qb, b, h);
  const int hk = h / (a.Hq / a.Hkv);
  const int q0_wg = qb * Tile::BQ;
  // This wavefront's queries.  T is a multiple of 128 but not necessarily of BQ: a wavefront past the
  // end works on the last 32 rows instead (it still takes part in the tile loads) and stores nothing.
  const bool live = q0_wg + wave * 32 < a.T;
  const int q0 = live ? q0_wg + wave * 32 : a.T - 32;

  // Q and dO fragments (B operands): lane (query l32, k-group g) holds d = 16kk + 8g .. +7.
  const __bf16* qp = (const __bf16*)a.q + b * a.qs.b + (int64_t)(q0 + l32) * a.qs.s + h * a.qs.h;
  const __bf16* dop = (const __bf16*)a.dout + b * a.dos.b + (int64_t)(q0 + l32) * a.dos.s + h * a.dos.h;
  bf16x8 qf[KK], dof[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) {
    qf[kk] = load8_within(qp, 16 * kk + 8 * g, a.d_real);
    dof[kk] = load8_within(dop, 16 * kk + 8 * g, a.d_real);
  }
  const int64_t stat_idx = ((int64_t)b * a.Hq + h) * a.T + q0 + l32;
  float off, delta;  // -lse * log2(e), rowsum(out * dO)
  if constexpr (FUSE_DELTA) {
    // The lane holds d = 16kk + 8g .. +7 of its query's dO; with the same pieces of out, the two lanes
    // of a query (g = 0, 1) each sum half of the row.
    const __bf16* op = (const __bf16*)a.out + b * a.os.b + (int64_t)(q0 + l32) * a.os.s + h * a.os.h;
    float part = 0.f;
#pragma unroll
    for (int kk = 0; kk < KK; kk++) {
      union {
        bf16x8 v;
        bf16x2 p[4];
      } o, d;
      o.v = load8_within(op, 16 * kk + 8 * g, a.d_real);
      d.v = dof[kk];
#pragma unroll
      for (int i = 0; i < 4; i++) part = E::dot2(o.p[i], d.p[i], part);
    }
    delta = xor32_sum(part);
    off = lse_to_exp2_offset(a.lse[stat_idx]);
    if (live && g == 0) {
      a.ndelta[stat_idx] = -delta;
      a.lse2[stat_idx] = off;
    }
  } else {
    off = a.lse2[stat_idx];
    delta = -a.ndelta[stat_idx];
  }
  const int qpos = q0 + l32 + a.q_off;
  const int qpos_min = q0 + a.q_off, qpos_max = q0 + 31 + a.q_off;  // of the wavefront
  int seg_q = 0;
  if (HAS_SEG) seg_q = a.seg[(int64_t)b * a.T + q0 + l32];

  // Keys that any query of this workgroup can see, widened to whole 64-key tiles (S is a multiple of
  // 128; the keys added by the widening are masked for every query).
  int k_begin = 0, k_end = a.S;
  if (a.mask_kind != AXL_MASK_NONE) {
    k_end = min(a.S, q0_wg + Tile::BQ + a.q_off);
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) k_begin = max(0, q0_wg + a.q_off - a.window);
  }
  // With segment ids: one pass over the ids of the key range shrinks it to the hull of the keys whose
  // id lies between the smallest and the largest id of this workgroup's queries, and records for
  // every 32-key sub-tile whether it carries a single id.
  __shared__ int s_sub[HAS_SEG ? kMaxSub : 1];
  int sub_g0 = 0;  // sub-tile that s_sub[0] describes
  if (HAS_SEG)
    sub_g0 = classify_segment_groups_tbl<64 * NW, Tile::BK>(a.seg_tbl + (int64_t)b * (a.T / kSegGroupRows),
                                                           q0_wg / kSegGroupRows, min(Tile::BQ, a.T - q0_wg) / kSegGroupRows, tid, k_begin,
                                                           k_end, s_sub, kMaxSub, kNotUniform);
  const int t_begin = k_begin / Tile::BK;
  const int trips = max(0, (k_end + Tile::BK - 1) / Tile::BK - t_begin);
  const int key0 = t_begin * Tile::BK;   // first key of sub-tile 0
  // keep(q, k)  <=>  (unsigned)(qpos - kpos) <= limit
  const unsigned limit = a.mask_kind == AXL_MASK_NONE             ? 0xffffffffu
                         : a.mask_kind == AXL_MASK_SLIDING_WINDOW ? (unsigned)a.window
                                                                  : 0x7fffffffu;

  floatx16 dq_acc[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq_acc[i][r] = 0.f;
  const float c = a.scale * kLog2e;

  // ---- tile loads: direct global->LDS, 1 KB (RPI rows) per instruction.  Wavefront w fetches rows
  // 16w .. 16w+15 of the K and of the V tile; lane l fills chunk slot l % CPR of row l / CPR with the
  // global chunk that the swizzle puts there.  Lanes 0..15 also fetch the 64 segment ids of the keys
  // (every wavefront issues that same load, so all wavefronts count the same loads in flight).
  constexpr int CPR = D / 8;  // 16-byte chunks per row
  constexpr int ROWS_PER_WAVE = Tile::BK / NW;
  constexpr bool PAIRS = Tile::DMA_PER_WAVE % 2 == 0;  // tile loads are issued in pairs when there are several
  unsigned k_lane[Tile::DMA_PER_WAVE], v_lane[Tile::DMA_PER_WAVE];  // byte offsets from the tile's first row
#pragma unroll
  for (int i = 0; i < Tile::DMA_PER_WAVE; i++) {
    const int row = ROWS_PER_WAVE * wave + Tile::RPI * i + lane / CPR;
    const int slot_chunk = (lane % CPR) ^ tile_swizzle<D>(row);
    const int chunk = slot_chunk * 8 < a.d_real ? slot_chunk : 0;
    // the second load of a pair carries an instruction offset of 1024, which also moves its source
    k_lane[i] = (unsigned)(row * (int)a.ks.s + chunk * 8) * 2 - (PAIRS ? (i % 2) * 1024 : 0);
    v_lane[i] = (unsigned)(row * (int)a.vs.s + chunk * 8) * 2 - (PAIRS ? (i % 2) * 1024 : 0);
  }
  const __bf16* k_src = (const __bf16*)a.k + b * a.ks.b + hk * a.ks.h + (int64_t)key0 * a.ks.s;
  const __bf16* v_src = (const __bf16*)a.v + b * a.vs.b + hk * a.vs.h + (int64_t)key0 * a.vs.s;
  // segment ids of the tile's 64 keys: lanes 0..15 fetch 4 ids each, from a scalar base
  const int32_t* s_src = HAS_SEG ? a.seg + (int64_t)b * a.T + key0 : nullptr;
  const unsigned s_lane = 16 * (lane & 15);
  const int64_t k_step = (int64_t)Tile::BK * a.ks.s, v_step = (int64_t)Tile::BK * a.vs.s;
  // The k-th group of loads (pairs of K loads, pairs of V loads, then the segment ids) of the cursor's
  // tile into the buffer at LDS address BUF_.
  constexpr int GRP_PER_TENSOR = PAIRS ? Tile::DMA_PER_WAVE / 2 : Tile::DMA_PER_WAVE;
  constexpr int NGRP = 2 * GRP_PER_TENSOR + (HAS_SEG ? 1 : 0);
#define AXL_DMA(BUF_, K_)                                                                          \
  {                                                                                               \
    constexpr int per_ = PAIRS ? 2 : 1;                                                           \
    if constexpr ((K_) < GRP_PER_TENSOR) {                                                        \
      const unsigned dst_ = (BUF_) + wave * (ROWS_PER_WAVE * Tile::ROWB) + per_ * (K_) * 1024;    \
      if constexpr (PAIRS) dma16x2(k_lane[(2 * (K_)) % Tile::DMA_PER_WAVE], k_lane[(2 * (K_) + 1) % Tile::DMA_PER_WAVE], k_src, dst_); \
      else dma16s(k_lane[(K_) % Tile::DMA_PER_WAVE], k_src, dst_);                                \
    } else if constexpr ((K_) < 2 * GRP_PER_TENSOR) {                                             \
      constexpr int kv_ = (K_) - GRP_PER_TENSOR;                                                  \
      const unsigned dst_ = (BUF_) + Tile::TILE_BYTES + wave * (ROWS_PER_WAVE * Tile::ROWB) + per_ * kv_ * 1024; \
      if constexpr (PAIRS) dma16x2(v_lane[(2 * kv_) % Tile::DMA_PER_WAVE], v_lane[(2 * kv_ + 1) % Tile::DMA_PER_WAVE], v_src, dst_); \
      else dma16s(v_lane[kv_ % Tile::DMA_PER_WAVE], v_src, dst_);                                 \
    } else {                                                                                      \
      /* no branch: the trip stays one scheduling region (all lanes are active here) */            \
      dma16s_first16(s_lane, s_src, (BUF_) + Tile::SEG_BASE);                                     \
    }                                                                                             \
  }
#define AXL_DMA_TILE(BUF_)                                                                         \
  {                                                                                               \
    AXL_DMA(BUF_, 0) AXL_DMA(BUF_, 1)                                                             \
    if constexpr (NGRP > 2) AXL_DMA(BUF_, 2)                                                      \
    if constexpr (NGRP > 3) AXL_DMA(BUF_, 3)                                                      \
    if constexpr (NGRP > 4) AXL_DMA(BUF_, 4)                                                      \
    static_assert(NGRP <= 5, "groups of tile loads");                                             \
  }
  // Prefetch cursor; it stops at the last tile (re-fetching that tile is harmless).
  int pf_idx = 0;
#define AXL_ADVANCE()                                                       \
  {                                                                         \
    const bool adv_ = pf_idx + 1 < trips;                                   \
    pf_idx += adv_ ? 1 : 0;                                                 \
    k_src += adv_ ? k_step : 0;                                             \
    v_src += adv_ ? v_step : 0;                                             \
    if (HAS_SEG) s_src += adv_ ? Tile::BK : 0;                              \
  }

  char* buf_b = smem;                         // tile t     (stage B reads)
  char* buf_a = smem + Tile::BUF_BYTES;       // tile t + 1 (stage A reads)
  char* buf_n = smem + 2 * Tile::BUF_BYTES;   // tile t + 2 (requested one trip ago, awaited at the end of this one)
  char* buf_s = smem + 3 * Tile::BUF_BYTES;   // tile t + 3 (requested during this trip)

  // Per-lane read offsets (bytes) into a swizzled tile.  Stage A: row swap_bits_2_3(l32), logical
  // chunk 2kk + g.  Stage B (transposing reads): row 8g + j16/4 (+4 for the second half, +16 for the
  // second group of 16 keys), logical byte column (16 half + 4 (j16 % 4)) * 2 + 64 dt.
  const int a_row = swap_bits_2_3(l32);
  const int a_row_off = a_row * Tile::ROWB;
  const int a_xor = tile_swizzle<D>(a_row) << 4;
  const int j16 = lane & 15, half = (lane >> 4) & 1;
  const int t_row = 8 * g + (j16 >> 2);
  const int t_col = (16 * half + 4 * (j16 & 3)) * 2;
  const int t_off0 = t_row * Tile::ROWB + (t_col & 15), t_off1 = t_off0 + 4 * Tile::ROWB;
  const int t_xor0 = tile_swizzle<D>(t_row) << 4, t_xor1 = tile_swizzle<D>(t_row + 4) << 4;
  int a_off[KK], tb_off[2][DT];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) a_off[kk] = a_row_off + ((kk * 32 + g * 16) ^ a_xor);
#pragma unroll
  for (int dt = 0; dt < DT; dt++) {
    tb_off[0][dt] = t_off0 + (((t_col & ~15) + dt * 64) ^ t_xor0);
    tb_off[1][dt] = t_off1 + (((t_col & ~15) + dt * 64) ^ t_xor1);
  }
  union TrFrag {
    bf16x8 v;
    shortx4 hlf[2];
  };
  // Stage-B fragment N_ = t8 * DT + dt of sub-tile SUB_ of the K tile whose per-lane addresses are
  // AD_: K^T rows 32dt .. 32dt+31 (head dim) by keys 16 t8 .. 16 t8 + 15 of the sub-tile.
#define AXL_B_READ_AT(AD_, SUB_, DST_, N_)                                       \
  {                                                                              \
    const int imm_ = (SUB_) * Tile::SUB_BYTES + 16 * ((N_) / DT) * Tile::ROWB;   \
    DST_.hlf[0] = lds_read_tr16(AD_[0][(N_) % DT] + imm_);                       \
    DST_.hlf[1] = lds_read_tr16(AD_[1][(N_) % DT] + imm_);                       \
  }

  union PackedOperand {
    bf16x8 v[2];
    bf16x2 p[8];
  };
  // Two register sets that swap roles from step to step: logits / dP of the sub-tile whose
  // elementwise stage is next, dS^T of the sub-tile whose stage B is next, segment ids.
  floatx16 s0, dp0, s1, dp1;
  PackedOperand ds0, ds1;
  intx4 sg0[4], sg1[4];
  // dP - delta comes out of the MFMA chain itself: the chain starts from -delta (the lane is a query,
  // so the 16 registers of its accumulator all start from the same value).
  floatx16 ndelta16;
#pragma unroll
  for (int r = 0; r < 16; r++) {
    s0[r] = s1[r] = 0.f;
    dp0[r] = dp1[r] = ndelta16[r] = -delta;
  }
  // Segment ids of sub-tile SUB_ of the tile in BUF_: register r of lane group g is key
  // 16(r/8) + 8g + (r%8) of the sub-tile.
#define AXL_READ_SEG_PART(BUF_, SUB_, T8_, SEG_)                                        \
  {                                                                                     \
    const char* st_ = (BUF_) + Tile::SEG_BASE + (SUB_) * 128 + 8 * g * 4;               \
    SEG_[2 * (T8_)] = *(const intx4*)(st_ + 64 * (T8_));                                \
    SEG_[2 * (T8_) + 1] = *(const intx4*)(st_ + 64 * (T8_) + 16);                       \
  }
  // Elementwise stage of element R_ of (S_, DP_) in three phases that the pipelined loop issues in
  // three consecutive MFMA slots, so that no instruction waits for the result of the one before it
  // (v_exp_f32 in particular has a long latency): exponent, exponential, product.  MASKED_ selects
  // the mask arithmetic; DIFF0_ is qpos - (first key of the sub-tile + 8g).
#define AXL_ELEM_1(S_, SEG_, DIFF0_, R_, MASKED_)                                              \
  {                                                                                            \
    const int r_ = (R_);                                                                       \
    float sv_ = S_[r_];                                                                        \
    if (MASKED_) {                                                                             \
      const unsigned diff_ = (unsigned)((DIFF0_) - (16 * (r_ / 8) + (r_ % 8)));                \
      sv_ = diff_ <= limit ? sv_ : kMasked;                                                    \
      if (HAS_SEG) sv_ = SEG_[r_ / 4][r_ % 4] == seg_q ? sv_ : kMasked;                        \
    }                                                                                          \
    S_[r_] = __builtin_fmaf(sv_, c, off);                                                      \
  }
#define AXL_ELEM_2(S_, R_) S_[R_] = fast_exp2(S_[R_]);
#define AXL_ELEM_3(S_, DP_, R_) DP_[R_] = S_[R_] * DP_[R_]; /* the dP chain started from -delta */
#define AXL_ELEM(S_, DP_, SEG_, DIFF0_, R_, MASKED_)                                           \
  {                                                                                            \
    AXL_ELEM_1(S_, SEG_, DIFF0_, R_, MASKED_)                                                  \
    AXL_ELEM_2(S_, R_)                                                                         \
    AXL_ELEM_3(S_, DP_, R_)                                                                    \
  }
  // Stage A of sub-tile SUB_ of the tile in BUF_ into (S_, DP_), not interleaved with anything
  // (pipeline fill).
#define AXL_STAGE_A_PLAIN(BUF_, SUB_, S_, DP_)                                                  \
  _Pragma("unroll") for (int kk = 0; kk < KK; kk++) {                                           \
    const bf16x8 ka_ = *(const bf16x8*)((BUF_) + (SUB_) * Tile::SUB_BYTES + a_off[kk]);         \
    const bf16x8 va_ = *(const bf16x8*)((BUF_) + Tile::TILE_BYTES + (SUB_) * Tile::SUB_BYTES + a_off[kk]); \
    S_ = E::mfma_32x32x16(ka_, qf[kk], S_);                     \
    DP_ = E::mfma_32x32x16(va_, dof[kk], DP_);                  \
  }

  constexpr int NS = NA + NB;          // MFMAs per step: stage B of sub-tile j, then stage A of sub-tile j+2
  constexpr int kAheadA = (NB < 6 ? NB : 6), kAheadB = (NB < 4 ? NB : 4);
  constexpr int NLD = Tile::DMA_PER_TILE;     // direct-to-LDS loads of a tile per wavefront
  constexpr int LD_SLOT0 = 2;                 // one per slot from here on, after the cursor moved in slot 1
  constexpr int LD_STRIDE = 2;                // a group of loads every other slot
  static_assert(LD_SLOT0 + LD_STRIDE * NGRP <= 2 * NS, "the loads of a tile fit into one trip");
  TrFrag bfr_next[kAheadB];            // first stage-B fragments of the next step
  const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  if (trips > 0) {
    // Everything the compiler tracks (stationary fragments, statistics) has landed before the first
    // untracked load, so its own wait counts never cover a tile load.
    wait_all_vmem();
    AXL_DMA_TILE(lds_address(buf_b))
    AXL_ADVANCE()
    AXL_DMA_TILE(lds_address(buf_a))
    AXL_ADVANCE()
    AXL_DMA_TILE(lds_address(buf_n))
    wait_all_vmem();  // tiles 0..2 have landed; nothing issued before the loop is pending
    __syncthreads();
    // Pipeline fill: stage A and the elementwise stage of sub-tile 0 (-> ds0), stage A of sub-tile 1
    // (-> s0, dp0), first stage-B fragments of sub-tile 0.
    AXL_STAGE_A_PLAIN(buf_b, 0, s1, dp1)
    if (HAS_SEG) {
      AXL_READ_SEG_PART(buf_b, 0, 0, sg1)
      AXL_READ_SEG_PART(buf_b, 0, 1, sg1)
    }
#pragma unroll
    for (int r = 0; r < 16; r++) AXL_ELEM(s1, dp1, sg1, qpos - 8 * g - key0, r, true)
#pragma unroll
    for (int i = 0; i < 8; i++) ds0.p[i] = E::pack(dp1[2 * i], dp1[2 * i + 1]);
    AXL_STAGE_A_PLAIN(buf_b, 1, s0, dp0)
    if (HAS_SEG) {
      AXL_READ_SEG_PART(buf_b, 1, 0, sg0)
      AXL_READ_SEG_PART(buf_b, 1, 1, sg0)
    }
    const char* p_ad[2][DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      p_ad[0][dt] = buf_b + tb_off[0][dt];
      p_ad[1][dt] = buf_b + tb_off[1][dt];
    }
#pragma unroll
    for (int i = 0; i < kAheadB; i++) AXL_B_READ_AT(p_ad, 0, bfr_next[i], i)
  }

  // One step (sub-tile j = 2t + H of the trip's tile): stage B of sub-tile j with DSB_, elementwise
  // stage of sub-tile j+1 from (S_E, DP_E, SEG_E) into DSB_N, stage A of sub-tile j+2 into
  // (S_A, DP_A), segment ids of sub-tile j+2 into SEG_N.  Sub-tile j is half H of the tile in buf_b,
  // sub-tile j+1 half 1-H of buf_b (H = 0) or half 0 of buf_a (H = 1), sub-tile j+2 half H of buf_a.
#define AXL_STEP(H_, MASKED_, S_E, DP_E, SEG_E, DSB_, DSB_N, S_A, DP_A, SEG_N)                          \
  {                                                                                                    \
    bf16x8 afr[NA];                                                                                    \
    TrFrag bfr[NB];                                                                                    \
    _Pragma("unroll") for (int i = 0; i < kAheadB; i++) bfr[i] = bfr_next[i];                          \
    const int diff0 = qpos - 8 * g - (key0 + (2 * t + (H_) + 1) * 32);                                 \
    __builtin_amdgcn_sched_barrier(0);                                                                 \
    _Pragma("unroll") for (int n = 0; n < NS; n++) {                                                   \
      /* ---- LDS fragments requested ahead of their MFMA */                                           \
      if (n + kAheadB < NB) AXL_B_READ_AT(b_ad, H_, bfr[n + kAheadB], n + kAheadB)                     \
      if (n + kAheadA >= NB && n + kAheadA - NB < NA) {                                                \
        const int x = n + kAheadA - NB;                                                                \
        afr[x] = *(const bf16x8*)(a_ad[x / 2] + (x % 2) * Tile::TILE_BYTES + (H_) * Tile::SUB_BYTES);  \
      }                                                                                                \
      /* ---- the MFMA of this slot.  Stage-B step m = t8 * DT + dt; stage-A step x: even -> S chain  \
         with K fragment x/2, odd -> dP chain with V fragment x/2. */                                  \
      if (n < NB) {                                                                                    \
        dq_acc[n % DT] = E::mfma_32x32x16(bfr[n].v, DSB_.v[n / DT], dq_acc[n % DT]); \
      } else {                                                                                         \
        const int x = n - NB;                                                                          \
        if (x % 2 == 0)                                                                                \
          S_A = E::mfma_32x32x16(afr[x], qf[x / 2], x == 0 ? zero16 : S_A); \
        else                                                                                           \
          DP_A = E::mfma_32x32x16(afr[x], dof[x / 2], x == 1 ? ndelta16 : DP_A); \
      }                                                                                                \
      /* ---- first stage-B fragments of sub-tile j+1 (read in the next step's first slots) */         \
      if (n >= NS - kAheadB) {                                                                         \
        if ((H_) == 0) AXL_B_READ_AT(b_ad, 1, bfr_next[n - (NS - kAheadB)], n - (NS - kAheadB))        \
        else AXL_B_READ_AT(n_ad, 0, bfr_next[n - (NS - kAheadB)], n - (NS - kAheadB))                  \
      }                                                                                                \
      /* ---- elementwise stage of sub-tile j+1: element e starts in slot e (NS-3)/16 and takes       \
         three slots; pairs are packed one slot after their second element is complete */              \
      _Pragma("unroll") for (int e = 0; e < 16; e++) {                                                 \
        if (e * (NS - 3) / 16 + 2 == n) AXL_ELEM_3(S_E, DP_E, e)                                       \
        if (e * (NS - 3) / 16 + 1 == n) AXL_ELEM_2(S_E, e)                                             \
        if (e * (NS - 3) / 16 == n) AXL_ELEM_1(S_E, SEG_E, diff0, e, MASKED_)                          \
      }                                                                                                \
      _Pragma("unroll") for (int i = 0; i < 8; i++)                                                    \
        if ((2 * i + 1) * (NS - 3) / 16 + 3 == n) DSB_N.p[i] = E::pack(DP_E[2 * i], DP_E[2 * i + 1]); \
      /* ---- tile t+3: advance the cursor, then one direct-to-LDS load per slot */                    \
      if ((H_) * NS + n == LD_SLOT0 - 1) AXL_ADVANCE()                                                 \
      if ((H_) * NS + n == LD_SLOT0) AXL_DMA(lds_s, 0)                                                 \
      if ((H_) * NS + n == LD_SLOT0 + LD_STRIDE) AXL_DMA(lds_s, 1)                                     \
      if (NGRP > 2 && (H_) * NS + n == LD_SLOT0 + 2 * LD_STRIDE) AXL_DMA(lds_s, 2 % NGRP)              \
      if (NGRP > 3 && (H_) * NS + n == LD_SLOT0 + 3 * LD_STRIDE) AXL_DMA(lds_s, 3 % NGRP)              \
      if (NGRP > 4 && (H_) * NS + n == LD_SLOT0 + 4 * LD_STRIDE) AXL_DMA(lds_s, 4 % NGRP)              \
      /* ---- segment ids of sub-tile j+2 for the next step's elementwise stage */                     \
      if (HAS_SEG && n == NS / 2) AXL_READ_SEG_PART(buf_a, H_, 0, SEG_N)                               \
      if (HAS_SEG && n == NS / 2 + 1) AXL_READ_SEG_PART(buf_a, H_, 1, SEG_N)                           \
      __builtin_amdgcn_sched_barrier(0);                                                               \
    }                                                                                                  \
  }

  // Trips [t_from, t_to); MASKED_C says whether their elementwise sub-tiles need mask arithmetic.
  // The loop is instantiated once per run of trips of one kind instead of branching inside one loop.
  auto run = [&](int t_from, int t_to, auto masked_c) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_c)::value;
    for (int t = t_from; t < t_to; t++) {
      const unsigned lds_s = lds_address(buf_s);
      const char* a_ad[KK];                // stage-A fragment addresses in tile t+1
      const char* b_ad[2][DT];             // stage-B fragment addresses in tile t
      const char* n_ad[2][DT];             // ... and in tile t+1, for the fragments read ahead of the next trip
#pragma unroll
      for (int kk = 0; kk < KK; kk++) a_ad[kk] = buf_a + a_off[kk];
#pragma unroll
      for (int dt = 0; dt < DT; dt++) {
        b_ad[0][dt] = buf_b + tb_off[0][dt];
        b_ad[1][dt] = buf_b + tb_off[1][dt];
        n_ad[0][dt] = buf_a + tb_off[0][dt];
        n_ad[1][dt] = buf_a + tb_off[1][dt];
      }
      AXL_STEP(0, MASKED, s0, dp0, sg0, ds0, ds1, s1, dp1, sg1)
      AXL_STEP(1, MASKED, s1, dp1, sg1, ds1, ds0, s0, dp0, sg0)
      // Tile t+2 (requested during the previous trip) has landed once at most this trip's loads are
      // outstanding; after the barrier every wavefront's part of it is visible, and nobody reads
      // tile t's buffer any more, which the next trip refills.
      wait_vmem_le<NLD>();
      __syncthreads();
      char* const tmp = buf_b;
      buf_b = buf_a;
      buf_a = buf_n;
      buf_n = buf_s;
      buf_s = tmp;
    }
  };
  // The elementwise sub-tiles of trip t are e = 2t + 1 and 2t + 2, starting at key key0 + 32 e.  Under
  // a sliding window the sub-tiles with qpos_max - k0 > window come first and need the mask; then
  // sub-tiles wholly visible to every query of the wavefront; from the first one with
  // k0 + 31 > qpos_min on, the causal mask.
  auto floor_div = [](int x, int y) { return x >= 0 ? x / y : -((-x + y - 1) / y); };
  int e0 = 0, e1 = 0x3fffffff;           // sub-tiles [e0, e1) need no mask
  if (a.mask_kind != AXL_MASK_NONE) {
    e1 = floor_div(qpos_min - 31 - key0, 32) + 1;
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) e0 = floor_div(qpos_max - a.window - key0 + 31, 32);
  }
  if (HAS_SEG) {
    // Sub-tiles whose 32 keys all carry the segment id that all 32 queries of this wavefront carry
    // need no segment mask either: take the first run [tA, tB) of such sub-tiles (the masked loop is
    // always correct, so whatever lies outside that run simply stays on it).
    const int nsub = 2 * trips;
    const int sub0 = key0 / 32 - sub_g0;  // table index of sub-tile 0
    int tA = 0, tB = 0;
    if (sub0 + nsub <= kMaxSub) {
      const int wq_id = __builtin_amdgcn_readfirstlane(seg_q);
      const bool q_uniform = __builtin_amdgcn_ballot_w64(seg_q != wq_id) == 0 && wq_id != kNotUniform;
      tA = tB = nsub;
      if (q_uniform) {
        for (int base = 0; base < nsub && tA == nsub; base += 64) {
          const int i = base + lane;
          const uint64_t m = __builtin_amdgcn_ballot_w64(i < nsub && s_sub[sub0 + min(i, nsub - 1)] == wq_id);
          if (m) tA = base + __builtin_ctzll(m);
        }
        for (int base = tA & ~63; base < nsub && tB == nsub; base += 64) {
          const int i = base + lane;
          const uint64_t m = __builtin_amdgcn_ballot_w64(i > tA && i < nsub && s_sub[sub0 + min(i, nsub - 1)] != wq_id);
          if (m) tB = base + __builtin_ctzll(m);
        }
      }
    }
    e0 = max(e0, tA);
    e1 = min(e1, tB);
    if (e1 <= e0) e0 = e1 = 0x3fffffff;
  }
  // trip t is unmasked iff 2t + 1 >= e0 and 2t + 2 < e1
  const int t0 = min(trips, max(0, e0 >= 0x3fffffff ? trips : floor_div(e0, 2)));
  const int t1 = min(trips, max(t0, e1 >= 0x3fffffff ? trips : floor_div(e1 - 3, 2) + 1));
  // On every path into the loops no compiler-tracked load is pending (the path with trips == 0 skips
  // the waits above): otherwise the compiler waits for "all loads" at the first use of a loaded
  // value inside the loops, which is a wait for the tile loads just issued.
  wait_all_vmem();
  run(0, t0, std::true_type{});
  run(t0, t1, std::false_type{});
  run(t1, trips, std::true_type{});
  // The cursor re-requests the last tile during the final trips (which keeps the count of
  // outstanding loads the same in every trip); none of those may still be in flight when this
  // workgroup's LDS is handed to the next one.
  wait_all_vmem();
#undef AXL_STEP
#undef AXL_READ_SEG_PART
#undef AXL_ELEM
#undef AXL_ELEM_1
#undef AXL_ELEM_2
#undef AXL_ELEM_3
#undef AXL_STAGE_A_PLAIN
#undef AXL_B_READ_AT
#undef AXL_DMA
#undef AXL_DMA_TILE
#undef AXL_ADVANCE

  if (!live) return;
  __bf16* dqp = (__bf16*)a.dq + b * a.dqs.b + (int64_t)(q0 + l32) * a.dqs.s + h * a.dqs.h;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int rq = 0; rq < 4; rq++) {
      union {
        bf16x2 p[2];
        uint2 u;
      } w;
      w.p[0] = E::pack(dq_acc[dt][4 * rq + 0] * a.scale, dq_acc[dt][4 * rq + 1] * a.scale);
      w.p[1] = E::pack(dq_acc[dt][4 * rq + 2] * a.scale, dq_acc[dt][4 * rq + 3] * a.scale);
      if (32 * dt + 8 * rq + 4 * g < a.d_real) *(uint2*)(dqp + 32 * dt + 8 * rq + 4 * g) = w.u;
    }
}

// Wavefronts per workgroup: at head_dim 64 the kernel fits 256 registers, and eight wavefronts (two per
// SIMD, 256 query rows share every K / V tile) are 4 % faster than four; at head_dim 128 they spill
// (+40 %).
template <typename E, int D, bool HAS_SEG, bool FUSE_DELTA>
static hipError_t launch_one(const BwdArgs& a, hipStream_t stream) {
  constexpr int NW = D == 64 ? 8 : 4;
  using Tile = DqRing<D, HAS_SEG, NW>;
  auto kernel = flash_bwd_dq_ring_kernel<E, D, HAS_SEG, NW, FUSE_DELTA>;
  hipError_t err = allow_dynamic_lds((const void*)kernel, Tile::LDS_BYTES);
  if (err != hipSuccess) return err;
  const int grid = ((a.T + Tile::BQ - 1) / Tile::BQ) * a.B * a.Hq;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(64 * NW), Tile::LDS_BYTES, stream, a);
  return hipGetLastError();
}

template <typename E>
static hipError_t launch_for(const BwdArgs& a, int head_dim, bool fuse_delta, hipStream_t stream) {
  const bool seg = a.seg != nullptr;
  if (fuse_delta) {
    if (head_dim == 128)
      return seg ? launch_one<E, 128, true, true>(a, stream) : launch_one<E, 128, false, true>(a, stream);
    return seg ? launch_one<E, 64, true, true>(a, stream) : launch_one<E, 64, false, true>(a, stream);
  }
  if (head_dim == 128)
    return seg ? launch_one<E, 128, true, false>(a, stream) : launch_one<E, 128, false, false>(a, stream);
  return seg ? launch_one<E, 64, true, false>(a, stream) : launch_one<E, 64, false, false>(a, stream);
}

hipError_t launch_bwd_dq(const BwdArgs& a, int dtype, int head_dim, bool fuse_delta, hipStream_t stream) {
  return dtype == AXL_F16 ? launch_for<ElemF16>(a, head_dim, fuse_delta, stream)
                          : launch_for<ElemBf16>(a, head_dim, fuse_delta, stream);
}

}  // namespace axl
