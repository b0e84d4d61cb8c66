// Flash-attention forward for gfx950.
//
// Replaces axlearn/common/flash_attention/gpu_attention.py:114-243 (`_mha_forward_kernel`) and its
// launcher (:293-425).  Same mathematics (FlashAttention-2 online softmax, fp32 statistics, P
// rounded to the value dtype before PV, out = acc / l, lse = m + log l) on a different machine
// mapping:
//
//   * one workgroup = 4 wavefronts = 128 query rows of one (batch, query head); each wavefront owns
//     32 query rows and keeps their Q fragments in registers for the whole kernel;
//   * K/V tiles of 64 keys are shared by the 4 wavefronts through LDS (double buffered); they arrive
//     by direct global->LDS loads, unpadded and XOR-swizzled, so no registers stage them;
//   * the S^T MFMAs of tile t+1 are interleaved with the exponentials of tile t, so the matrix pipe
//     works through the softmax of the wavefront that feeds it;
//   * the logits are produced TRANSPOSED, S^T = K Q^T, with v_mfma_f32_32x32x16_bf16: a lane then
//     owns one query column and 16 keys per 32-key sub-tile, so the softmax row statistics are
//     in-register reductions plus a single exchange with lane^32, and exp(S^T) is already in the
//     B-operand layout of the second MFMA, O^T += V^T P^T: P never touches LDS;
//   * V^T fragments come from the row-major V tile through the transposing LDS read
//     (ds_read_b64_tr_b16);
//   * GQA reads the shared kv head directly (no repeated KV in HBM), and workgroups that share a kv
//     head are placed on the same XCD so its L2 serves the re-reads.
#include <type_traits>

#include <cstdlib>

#include "common.h"

namespace axl {

struct FwdArgs {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse;
  const int32_t* seg;
  const float* sink;  // [Hq] logit of the per-head attention sink, or nullptr
  const int32_t* q_offs;  // [B] per-sequence addition to q_off, or nullptr
  AuxArgs aux;        // dense bias / dropout mask (read only by the AUX instantiations)
  Strides3 qs, ks, vs, os;
  int B, T, S, Hq, Hkv;
  int mask_kind, window, q_off;
  float scale;
  int d_real;  // head_dim of the tensors: a multiple of 8, at most the compiled width D (16-bit kernels)
};

// NW wavefronts of 32 query rows each.  The kernels are launched with 4 (two workgroups per CU); 8
// (one workgroup per CU, twice as many query rows sharing every K / V tile that comes in from L2) was
// measured and is not used: -4 % on causal MHA at 8192 tokens, +1 to +3 % on the GQA and windowed shapes.
template <int D, int NW = 4>
struct FwdTile {
  static constexpr int BQ = 32 * NW;          // query rows per workgroup
  static constexpr int BK = 64;               // keys per LDS tile
  static constexpr int ROWB = D * 2;          // bytes per K / V row in LDS: unpadded
  static constexpr int TILE_BYTES = BK * ROWB;
  static constexpr int NSEG = 4;              // ring of segment-id rows (a tile's ids outlive its K buffer)
  static constexpr int SEG_BASE = 4 * TILE_BYTES;            // {K, V} x double buffer, then the ids
  static constexpr int LDS_BYTES = SEG_BASE + NSEG * BK * 4;
  static constexpr int WROWS = BK / NW;       // tile rows that one wavefront fetches
  static constexpr int DMA_PER_WAVE = TILE_BYTES / 1024 / NW;  // direct-to-LDS loads per wavefront per tile
  // Tiles arrive by direct global->LDS loads: unpadded rows, chunks XOR-swizzled (tile_swizzle).
  __device__ static __forceinline__ int swz(int row) { return tile_swizzle<D>(row); }
};

constexpr int kMaxSegTiles = 1024;               // key tiles whose segment ids the forward classifies
constexpr int kSegNotUniform = -0x7fffffff - 1;  // marks a tile with more than one segment id

template <typename E, int D, bool AUX, int NW = 4>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(AUX ? 1 : 2, AUX ? 1 : 2)))
void flash_fwd_kernel(const FwdArgs a) {
  using Tile = FwdTile<D, NW>;
  constexpr int KK = D / 16;  // MFMA k-steps over head_dim
  constexpr int DT = D / 32;  // 32-row output tiles over head_dim
  constexpr int CPR = D / 8;  // 16-byte chunks per row
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* const k_lds = smem;
  char* const v_lds = smem + 2 * Tile::TILE_BYTES;
  char* const seg_lds = smem + Tile::SEG_BASE;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  int qb, b, h;
  decode_block(blockIdx.x, a.T / Tile::BQ, a.B, a.Hq, a.Hkv, 256 / NW, qb, b, h);
  const int hk = h / (a.Hq / a.Hkv);
  const int q_off = a.q_off + (a.q_offs ? a.q_offs[b] : 0);  // position of this sequence's query row 0
  const int q0_wg = qb * Tile::BQ;
  const int q0 = q0_wg + wave * 32;

  const __bf16* qp = (const __bf16*)a.q + b * a.qs.b + (int64_t)(q0 + l32) * a.qs.s + h * a.qs.h;
  const __bf16* kp = (const __bf16*)a.k + b * a.ks.b + hk * a.ks.h;
  const __bf16* vp = (const __bf16*)a.v + b * a.vs.b + hk * a.vs.h;

  // Q fragments: B operand of S^T = K Q^T; lane (query l32, k-group g) holds d = 16kk + 8g .. +7.
  // (A head_dim below the compiled width: the columns past it are zeros here, so whatever the K tile
  // holds in them adds nothing to the logits; the V columns past it make output columns that are not
  // stored.  The tiles fetch slice 0 of the row in their place: finite values, no padded copies.)
  bf16x8 qf[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) {
    const bf16x8 zero8 = {};
    qf[kk] = 16 * kk + 8 * g < a.d_real ? *(const bf16x8*)(qp + 16 * kk + 8 * g) : zero8;
  }

  // Visible key range of this workgroup.
  int k_begin = 0, k_end = a.S;
  if (a.mask_kind != AXL_MASK_NONE) {
    k_end = min(a.S, q0_wg + Tile::BQ + q_off);
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) k_begin = max(0, q0_wg + q_off - a.window);
  }
  const int seg_q = a.seg ? a.seg[(int64_t)b * a.T + q0 + l32] : 0;
  const int32_t* seg_k = a.seg ? a.seg + (int64_t)b * a.T : nullptr;
  // With segment ids: one pass over the ids of the key range shrinks it to the hull of the keys whose
  // id lies between the smallest and the largest id of this workgroup's queries, and records for
  // every 64-key tile whether it carries a single id.  A tile whose keys all carry the one id that
  // all 32 queries of a wavefront carry needs no segment mask.
  __shared__ int s_tile_id[kMaxSegTiles];
  int seg_t0 = 0;          // tile that s_tile_id[0] describes
  if (seg_k) seg_t0 = classify_segment_groups<Tile::BK, 64 * NW>(seg_q, seg_k, tid, k_begin, k_end, s_tile_id, kMaxSegTiles,
                                                            kSegNotUniform);
  const int t_begin = k_begin / Tile::BK;
  const int t_end = (k_end + Tile::BK - 1) / Tile::BK;
  bool seg_fast = false;   // this wavefront's queries share one id and the table covers the tiles
  int wq_id = 0;
  if (seg_k && t_end - seg_t0 <= kMaxSegTiles) {
    wq_id = __builtin_amdgcn_readfirstlane(seg_q);
    seg_fast = __builtin_amdgcn_ballot_w64(seg_q != wq_id) == 0 && wq_id != kSegNotUniform;
  }

  // Dense bias / dropout mask rows of this lane's query (AUX instantiation only).  The bias joins
  // the raw logits as bias / scale, so the scale folded into the exponent applies to both.
  const char* bias_row = nullptr;
  const uint8_t* drop_row = nullptr;
  if constexpr (AUX) {
    if (a.aux.bias) bias_row = a.aux.bias + b * a.aux.bias_sb + h * a.aux.bias_sh + (int64_t)(q0 + l32) * a.aux.bias_sr;
    if (a.aux.drop) drop_row = a.aux.drop + b * a.aux.drop_sb + h * a.aux.drop_sh + (int64_t)(q0 + l32) * a.aux.drop_sr;
  }
  const int qpos = q0 + l32 + q_off;       // this lane's query position
  const int qpos_min = q0 + q_off, qpos_max = q0 + 31 + q_off;  // of the wavefront
  // Tiles this wavefront has to process (the others it only helps to load): [tw_begin, tw_end).
  int tw_begin = t_begin, tw_end = t_end;
  if (a.mask_kind != AXL_MASK_NONE) {
    tw_end = min(t_end, qpos_max / Tile::BK + 1);
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) tw_begin = max(t_begin, (qpos_min - a.window) / Tile::BK);
    tw_begin = max(tw_begin, t_begin);
  }

  floatx16 o[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[i][r] = 0.f;
  float m_run = kNegInf;  // running row max of the raw (unscaled) logits
  float l_run = 0.f;      // this lane's share of the running row sum (lanes l and l^32 split it)
  const float c = a.scale * kLog2e;
  if (a.sink) {
    // The sink is one more logit per row, with no value row (attention.py:608-626): it enters the
    // running softmax state as an already-processed key of weight exp(sink - m) = 1.
    m_run = a.sink[h] / a.scale;
    l_run = g == 0 ? 1.f : 0.f;
  }

  // ---- tile loads: wavefront w fetches rows 16w .. 16w+15 of a K (or V) tile, 1 KB per
  // instruction (1024 / ROWB rows); lane l's chunk slot is l % CPR of row l / CPR.
  constexpr int RPI = 1024 / Tile::ROWB;  // rows per instruction
  static_assert(Tile::DMA_PER_WAVE % 2 == 0, "tile loads are issued in pairs");
  unsigned k_src[Tile::DMA_PER_WAVE], v_src[Tile::DMA_PER_WAVE];  // byte offsets from the tile's first row
#pragma unroll
  for (int i = 0; i < Tile::DMA_PER_WAVE; i++) {
    const int row = Tile::WROWS * wave + RPI * i + lane / CPR;
    const int slot_chunk = (lane % CPR) ^ Tile::swz(row);
    const int chunk = slot_chunk * 8 < a.d_real ? slot_chunk : 0;
    // the second load of a pair carries an instruction offset of 1024, which also moves its source
    k_src[i] = (unsigned)(row * (int)a.ks.s + chunk * 8) * 2 - (i % 2) * 1024;
    v_src[i] = (unsigned)(row * (int)a.vs.s + chunk * 8) * 2 - (i % 2) * 1024;
  }
  const unsigned lds0 = lds_address(smem);
  auto issue_k = [&](int t, int buf) {
    const __bf16* src = kp + (int64_t)t * Tile::BK * a.ks.s;
    const unsigned dst = lds0 + buf * Tile::TILE_BYTES + wave * (Tile::WROWS * Tile::ROWB);
#pragma unroll
    for (int i = 0; i < Tile::DMA_PER_WAVE; i += 2) dma16x2(k_src[i], k_src[i + 1], src, dst + i * 1024);
    if (seg_k && wave == 0 && lane < Tile::BK / 4)  // 64 ids = 16 lanes x 16 bytes
      dma16(seg_k + t * Tile::BK + 4 * lane, lds0 + Tile::SEG_BASE + (t % Tile::NSEG) * (Tile::BK * 4));
  };
  // One pair of a tile's loads (FAST tiles deal the pairs out over their MFMA slots).
  auto issue_k_pair = [&](int t, int buf, int i) __attribute__((always_inline)) {
    const __bf16* src = kp + (int64_t)t * Tile::BK * a.ks.s;
    dma16x2(k_src[i], k_src[i + 1], src, lds0 + buf * Tile::TILE_BYTES + wave * (Tile::WROWS * Tile::ROWB) + i * 1024);
  };
  auto issue_v_pair = [&](int t, int buf, int i) __attribute__((always_inline)) {
    const __bf16* src = vp + (int64_t)t * Tile::BK * a.vs.s;
    dma16x2(v_src[i], v_src[i + 1], src, lds0 + (2 + buf) * Tile::TILE_BYTES + wave * (Tile::WROWS * Tile::ROWB) + i * 1024);
  };
  auto issue_v = [&](int t, int buf) {
    const __bf16* src = vp + (int64_t)t * Tile::BK * a.vs.s;
    const unsigned dst = lds0 + (2 + buf) * Tile::TILE_BYTES + wave * (Tile::WROWS * Tile::ROWB);
#pragma unroll
    for (int i = 0; i < Tile::DMA_PER_WAVE; i += 2) dma16x2(v_src[i], v_src[i + 1], src, dst + i * 1024);
  };

  // ---- per-lane LDS read offsets (bytes).  K row reads: row swap_bits_2_3(l32) (+32 per sub-tile),
  // logical chunk 2kk + g.  V transposing reads: row 8g + j16/4 (+4 for the second half, +16 per
  // 16-key group), logical byte column (16 half + 4 (j16 % 4)) * 2 + 64 dt.
  const int k_row = swap_bits_2_3(l32);
  const int k_row_off = k_row * Tile::ROWB;
  const int k_xor = Tile::swz(k_row) << 4;
  const int j16 = lane & 15, half = (lane >> 4) & 1;
  const int v_row = 8 * g + (j16 >> 2);
  const int v_col = (16 * half + 4 * (j16 & 3)) * 2;
  const int v_off0 = v_row * Tile::ROWB + (v_col & 15), v_off1 = v_off0 + 4 * Tile::ROWB;
  const int v_xor0 = Tile::swz(v_row) << 4, v_xor1 = Tile::swz(v_row + 4) << 4;

  // Everything the compiler tracks (Q, segment ids) has landed before the first untracked load.
  wait_all_vmem();
  if (t_begin < t_end) {
    issue_k(t_begin, 0);
    issue_v(t_begin, 0);
    if (t_begin + 1 < t_end) issue_k(t_begin + 1, 1);
  }

  union VFrag {
    bf16x8 v;
    shortx4 hlf[2];
  };
  // Logits of the tile whose softmax is next (sub-tile ks holds keys 32ks .. 32ks+31) and of the tile
  // after it: two register sets that swap roles from tile to tile, so nothing is copied.
  floatx16 s_even[2], s_odd[2];
#define AXL_K_FRAG(KT_, KK_, KS_) \
  (*(const bf16x8*)((KT_) + (KS_) * 32 * Tile::ROWB + k_row_off + ((((KK_) * 32) + g * 16) ^ k_xor)))
  // S^T of one tile, nothing interleaved (pipeline fill).
#define AXL_S_PLAIN(KT_, S_)                                                                         \
  {                                                                                                  \
    _Pragma("unroll") for (int ks = 0; ks < 2; ks++)                                                 \
      _Pragma("unroll") for (int r = 0; r < 16; r++) S_[ks][r] = 0.f;                                \
    _Pragma("unroll") for (int kk = 0; kk < KK; kk++)                                                \
      _Pragma("unroll") for (int ks = 0; ks < 2; ks++)                                               \
        S_[ks] = E::mfma_32x32x16(AXL_K_FRAG(KT_, kk, ks), qf[kk], S_[ks]); \
  }

  // AUX: raw bias words and dropout bytes of the lane's 4 runs of 8 keys, requested one tile ahead
  // with ordinary (compiler-tracked) loads.  Run i covers keys 32(i/2) + 16(i%2) + 8g .. +7 of the tile;
  // an fp32 bias fills both vectors of a run, a bf16 bias the first.
  u32x4 bias_nx[AUX ? 8 : 1];
  uint2 drop_nx[AUX ? 4 : 1];
  // Both tests are uniform (the row pointers are not: they differ by lane).  A bf16 bias repeats its
  // one load so that the request is the same straight-line code for both element types.
  const bool has_bias = AUX && a.aux.bias != nullptr, has_drop = AUX && a.aux.drop != nullptr;
  const int bias_shift = a.aux.bias_f32 ? 2 : 1, bias_second = a.aux.bias_f32 ? 16 : 0;
  auto aux_request = [&](int t) __attribute__((always_inline)) {
    if constexpr (AUX) {
      const int k0 = t * Tile::BK + 8 * g;
      if (has_bias) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const char* p = bias_row + ((int64_t)(k0 + 32 * (i / 2) + 16 * (i % 2)) << bias_shift);
          bias_nx[2 * i] = *(const u32x4*)p;
          bias_nx[2 * i + 1] = *(const u32x4*)(p + bias_second);
        }
      }
      if (has_drop) {
#pragma unroll
        for (int i = 0; i < 4; i++) drop_nx[i] = *(const uint2*)(drop_row + k0 + 32 * (i / 2) + 16 * (i % 2));
      }
    }
  };
  if (t_begin < t_end && t_begin >= tw_begin && t_begin < tw_end) aux_request(t_begin);

  // Pipeline fill: S^T of the first tile.
  wait_vmem_le<0>();
  __syncthreads();
  if (t_begin < t_end && t_begin >= tw_begin && t_begin < tw_end) AXL_S_PLAIN(k_lds, s_even)

  // One tile: softmax and P V of tile t (logits in s), S^T of tile t+1 (into s_nxt).  buf_c is the
  // parity of the tile, i.e. which half of the double buffers holds it.
  // Lane-local maximum of the logits that the last FAST tile left in its s_nxt (taken between its P V
  // MFMAs); a FAST tile starts from it instead of scanning its 32 logits.
  float mx_carry = kNegInf;
  auto tile_step = [&](int t, auto buf_c, floatx16 (&s)[2], floatx16 (&s_nxt)[2], auto fast_c) __attribute__((always_inline)) {
    constexpr int buf = decltype(buf_c)::value;
    // FAST: a tile in the interior of this wavefront's range - its softmax needs no mask of any kind
    // and the tile after it is processed too - so every test below is decided at compile time.
    constexpr bool FAST = decltype(fast_c)::value;
    // K(t+1) and V(t) (requested one iteration ago) become visible to the whole workgroup and every
    // wavefront is done with S(t) and PV(t-1); the buffers those were read from are then refilled
    // with K(t+2) and V(t+1).
    wait_vmem_le<0>();
    __syncthreads();
    // FAST tiles issue the tile loads one pair per MFMA slot further down, where their issue time
    // overlaps the matrix pipe's work; K(t+2) may not exist (t + 2 == t_end), then the last tile is
    // fetched again into a buffer that nobody reads any more.
    const int t_k2 = min(t + 2, t_end - 1);

    const bool do_sm = FAST || (t >= tw_begin && t < tw_end);          // softmax and PV of tile t
    const bool do_s = FAST || (t + 1 >= tw_begin && t + 1 < tw_end);   // S of tile t + 1
    // Bias and dropout bytes of tile t arrived with the wait above (they were requested one tile
    // ago, ahead of that tile's K / V loads); they are consumed here, before anything else is
    // requested, so the compiler's own wait for them finds the counter at zero already.
    uint2 dm[2][2] = {};  // dropout bytes of the lane's 4 runs of 8 keys
    if constexpr (AUX && !FAST) {
      if (do_sm) {
        if (has_bias) {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            float bv[8];
            if (a.aux.bias_f32) {
#pragma unroll
              for (int j = 0; j < 4; j++) {
                // (copies first: a bit cast applied to the vector element itself reads element 0)
                const unsigned w0 = bias_nx[2 * i][j], w1 = bias_nx[2 * i + 1][j];
                bv[j] = __builtin_bit_cast(float, w0);
                bv[4 + j] = __builtin_bit_cast(float, w1);
              }
            } else {
#pragma unroll
              for (int j = 0; j < 4; j++) {
                bv[2 * j] = __builtin_bit_cast(float, bias_nx[2 * i][j] << 16);
                bv[2 * j + 1] = __builtin_bit_cast(float, bias_nx[2 * i][j] & 0xffff0000u);
              }
            }
#pragma unroll
            for (int j = 0; j < 8; j++)
              s[i / 2][8 * (i % 2) + j] = __builtin_fmaf(bv[j], a.aux.inv_scale, s[i / 2][8 * (i % 2) + j]);
          }
        }
        if (has_drop) {
#pragma unroll
          for (int i = 0; i < 4; i++) dm[i / 2][i % 2] = drop_nx[i];
        }
      }
      if (do_s) aux_request(t + 1);
    }
    if constexpr (!FAST) {
      if (t + 2 < t_end) issue_k(t + 2, buf);
      if (t + 1 < t_end) issue_v(t + 1, buf ^ 1);
    }
    const char* kt = k_lds + (buf ^ 1) * Tile::TILE_BYTES;   // K(t+1)
    const char* vt = v_lds + buf * Tile::TILE_BYTES;         // V(t)
    const int k0 = t * Tile::BK;
    if (!do_sm) {
      if (do_s) AXL_S_PLAIN(kt, s_nxt)
      return;
    }

    // ---- masks of tile t.  Register r of sub-tile ks in lane group g is key k0 + 32ks + 16(r/8) + 8g + (r%8).
    // Probability that enters P V: zero where the dropout mask says so (the row sum keeps it).
    auto after_dropout = [&](int idx, float p) {
      if constexpr (AUX) {
        const int ks = idx / 16, r = idx % 16;
        const unsigned w = (r % 8) < 4 ? dm[ks][r / 8].x : dm[ks][r / 8].y;
        return ((w >> (8 * (r % 4))) & 0xffu) ? 0.f : p;
      } else {
        return p;
      }
    };
    bool need_mask = false;
    const unsigned mask_limit = a.mask_kind == AXL_MASK_SLIDING_WINDOW ? (unsigned)a.window : 0x7fffffffu;
    if (!FAST && a.mask_kind != AXL_MASK_NONE) {
      need_mask = k0 + Tile::BK - 1 > qpos_min;
      if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) need_mask = need_mask || (qpos_max - k0 > a.window);
    }
    if (need_mask) {
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        const int diff0 = qpos - (k0 + 32 * ks + 8 * g);  // qpos - kpos for r == 0
#pragma unroll
        for (int r = 0; r < 16; r++) {
          // keep(q, k)  <=>  0 <= qpos - kpos <= window: one unsigned comparison, one select
          const unsigned diff = (unsigned)(diff0 - (16 * (r / 8) + (r % 8)));
          s[ks][r] = diff <= mask_limit ? s[ks][r] : kMasked;
        }
      }
    }
    if (!FAST && seg_k && !(seg_fast && s_tile_id[t - seg_t0] == wq_id)) {
      const char* sg = seg_lds + (t % Tile::NSEG) * (Tile::BK * 4);
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
#pragma unroll
        for (int t8 = 0; t8 < 2; t8++) {
          const intx4 s0 = *(const intx4*)(sg + (32 * ks + 16 * t8 + 8 * g) * 4);
          const intx4 s1 = *(const intx4*)(sg + (32 * ks + 16 * t8 + 8 * g) * 4 + 16);
#pragma unroll
          for (int j = 0; j < 4; j++) {
            s[ks][8 * t8 + j] = (s0[j] == seg_q) ? s[ks][8 * t8 + j] : kMasked;
            s[ks][8 * t8 + 4 + j] = (s1[j] == seg_q) ? s[ks][8 * t8 + 4 + j] : kMasked;
          }
        }
      }
    }

    // ---- row maximum and (lazy) rescaling.  The running max, and with it the accumulators, only
    // moves when the new max exceeds it by more than 2^kLazyLog2 in the exponent; until then exp2 is
    // taken against the stale max, which scales numerator and denominator alike.
    float mx = m_run;
    if constexpr (FAST) {
      mx = fmaxf(mx, mx_carry);
    } else {
#pragma unroll
      for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[ks][r]);
    }
    mx = xor32_max(mx);
    constexpr float kLazyLog2 = 8.0f;
    const bool move = (mx - m_run) * c > kLazyLog2;
    if (__builtin_amdgcn_ballot_w64(move) != 0) {
      // Subtract first: (m_run * c - mx * c) would be contracted into an fma whose result, for
      // equal maxima, is the rounding error of the product instead of an exact 0.
      const float corr = move ? fast_exp2((m_run - mx) * c) : 1.0f;
      m_run = move ? mx : m_run;
      l_run *= corr;
#pragma unroll
      for (int i = 0; i < DT; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[i][r] *= corr;
    }
    const float mc = m_run * c;

    // ---- exp2 of tile t, interleaved with the S^T MFMAs of tile t+1: slot n runs MFMA (kk, ks) =
    // (n / 2, n % 2) and the exponentials of 32 / (2 KK) elements; LDS fragments are requested
    // kAhead slots ahead.
    constexpr int NSL = 2 * KK, EPS = 32 / NSL, kAhead = 6;
    static_assert(NSL * EPS == 32, "elements must tile the MFMA slots");
    float lsum = 0.f;
    union {
      bf16x8 v[4];
      bf16x2 p[16];
    } pb;
    if (do_s) {
      bf16x8 kfr[NSL];
#pragma unroll
      for (int n = 0; n < (kAhead < NSL ? kAhead : NSL); n++) kfr[n] = AXL_K_FRAG(kt, n / 2, n % 2);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int n = 0; n < NSL; n++) {
        if (n + kAhead < NSL) kfr[n + kAhead] = AXL_K_FRAG(kt, (n + kAhead) / 2, (n + kAhead) % 2);
        if constexpr (FAST) {
          constexpr int kPairs = Tile::DMA_PER_WAVE / 2;
          if (n % 2 == 0 && n / 2 < kPairs) issue_k_pair(t_k2, buf, n);
          if (n % 2 == 0 && n / 2 >= kPairs && n / 2 < 2 * kPairs) issue_v_pair(t + 1, buf ^ 1, n - 2 * kPairs);
          // the ids of tile t+2 for a general tile that may follow (every wavefront fetches the same
          // 256 bytes: no branch on the wavefront number inside the slot sequence)
          if (n == 4 * kPairs && seg_k)
            dma16s_first16(16 * (lane & 15), seg_k + t_k2 * Tile::BK, lds0 + Tile::SEG_BASE + (t_k2 % Tile::NSEG) * (Tile::BK * 4));
          // The chain in vector registers where the next tile's softmax reads it, started from a
          // literal zero: no register is cleared and none is copied.  (The 16 P V MFMAs of this tile lie
          // between the end of the chain and the first read of its result.)
          if (n < 2) E::mfma_32x32x16_vgpr_zero(kfr[n], qf[n / 2], s_nxt[n % 2]);
          else E::mfma_32x32x16_vgpr(kfr[n], qf[n / 2], s_nxt[n % 2]);
        } else if (n < 2) {
          const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          s_nxt[n % 2] = E::mfma_32x32x16(kfr[n], qf[n / 2], zero16);
        } else {
          s_nxt[n % 2] = E::mfma_32x32x16(kfr[n], qf[n / 2], s_nxt[n % 2]);
        }
#pragma unroll
        for (int e = 0; e < EPS; e++) {
          const int idx = n * EPS + e;
          const float p = fast_exp2(__builtin_fmaf(s[idx / 16][idx % 16], c, -mc));
          lsum += p;
          const float pu = after_dropout(idx, p);
          s[idx / 16][idx % 16] = pu;
          if (idx % 2 == 1) pb.p[idx / 2] = E::pack(s[idx / 16][idx % 16 - 1], pu);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int idx = 0; idx < 32; idx++) {
        const float p = fast_exp2(__builtin_fmaf(s[idx / 16][idx % 16], c, -mc));
        lsum += p;
        const float pu = after_dropout(idx, p);
        s[idx / 16][idx % 16] = pu;
        if (idx % 2 == 1) pb.p[idx / 2] = E::pack(s[idx / 16][idx % 16 - 1], pu);
      }
    }
    l_run += lsum;

    // ---- O^T += V^T P^T, software pipelined: each MFMA issues together with the transposing reads
    // of the step kPvAhead ahead of it.  PV step n = (ks*2 + t8)*DT + dt multiplies
    // V^T[32dt.., keys 32ks+16t8..] with P^T.
    constexpr int kPvSteps = 4 * DT, kPvAhead = 4;
    VFrag vfr[kPvSteps];
#define AXL_PV_READ(N_)                                                                                  \
  {                                                                                                      \
    const char* va_ = vt + (16 * ((N_) / DT)) * Tile::ROWB;                                              \
    vfr[N_].hlf[0] = lds_read_tr16(va_ + v_off0 + (((v_col & ~15) + ((N_) % DT) * 64) ^ v_xor0));        \
    vfr[N_].hlf[1] = lds_read_tr16(va_ + v_off1 + (((v_col & ~15) + ((N_) % DT) * 64) ^ v_xor1));        \
  }
#pragma unroll
    for (int n = 0; n < kPvAhead; n++) AXL_PV_READ(n)
    __builtin_amdgcn_sched_barrier(0);
    float pm[4] = {kMasked, kMasked, kMasked, kMasked};
#pragma unroll
    for (int n = 0; n < kPvSteps; n++) {
      if (n + kPvAhead < kPvSteps) AXL_PV_READ(n + kPvAhead)
      o[n % DT] = E::mfma_32x32x16(vfr[n].v, pb.v[n / DT], o[n % DT]);
      if constexpr (FAST) {
        // Row maximum of the next tile's logits, two per slot from slot 2 on: by then two MFMAs have
        // been issued after the last one of the S chains, whose results these reads therefore find
        // complete.  Four independent partial maxima keep the chains short.
#pragma unroll
        for (int j = 0; j < 16; j++)
          if (2 + j * (kPvSteps - 2) / 16 == n)
            pm[j % 4] = fmaxf(fmaxf(pm[j % 4], s_nxt[(2 * j) / 16][(2 * j) % 16]), s_nxt[(2 * j + 1) / 16][(2 * j + 1) % 16]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (FAST) mx_carry = fmaxf(fmaxf(pm[0], pm[1]), fmaxf(pm[2], pm[3]));
#undef AXL_PV_READ
  };
  {
    // Tiles [f_lo, f_hi) of this wavefront take the FAST form: inside its own range, the tile after
    // them inside it too, no positional mask (every key of the tile at or before the wavefront's first
    // query and, under a sliding window, within the window of its last query), no segment ids, no bias
    // or dropout mask.  f_lo has the parity of t_begin so that a pair of FAST tiles uses the register
    // sets and the buffers in the order (even, odd).
    const std::integral_constant<int, 0> c0{};
    const std::integral_constant<int, 1> c1{};
    int f_lo = t_end, f_hi = t_end;
    if (!AUX && (!seg_k || seg_fast)) {
      f_lo = tw_begin;
      f_hi = tw_end - 1;
      if (a.mask_kind != AXL_MASK_NONE) {
        f_hi = min(f_hi, qpos_min >= Tile::BK - 1 ? (qpos_min - (Tile::BK - 1)) / Tile::BK + 1 : 0);
        if (a.mask_kind == AXL_MASK_SLIDING_WINDOW)
          f_lo = max(f_lo, qpos_max - a.window > 0 ? (qpos_max - a.window + Tile::BK - 1) / Tile::BK : 0);
      }
      if (seg_k) {
        // ... and, with segment ids, only the run of tiles that ends at f_hi and whose keys all carry the
        // one id that all of this wavefront's queries carry (lane j looks at tile base - j; the lowest
        // set bit of the ballot is the last tile that breaks the run).
        for (int base = f_hi - 1; base >= f_lo; base -= 64) {
          const int i = base - lane;
          const uint64_t m = __builtin_amdgcn_ballot_w64(i >= f_lo && s_tile_id[i - seg_t0] != wq_id);
          if (m) {
            f_lo = base - __builtin_ctzll(m) + 1;
            break;
          }
        }
      }
      f_lo += (f_lo - t_begin) & 1;
    }
    int t = t_begin;
    // Pairs of tiles in the general form up to tile t_to (t and t_to have the parity of t_begin).
    auto generic_pairs_to = [&](int t_to) __attribute__((always_inline)) {
      for (; t + 1 < t_to; t += 2) {
        tile_step(t, c0, s_even, s_odd, std::false_type{});
        tile_step(t + 1, c1, s_odd, s_even, std::false_type{});
      }
    };
    if constexpr (!AUX) {
      generic_pairs_to(min(f_lo, t_end));
      if (t + 1 < f_hi) {  // the first FAST tile's lane-local maximum (later ones get theirs from the tile before)
        mx_carry = kMasked;
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
          for (int r = 0; r < 16; r++) mx_carry = fmaxf(mx_carry, s_even[ks][r]);
      }
      for (; t + 1 < f_hi; t += 2) {
        tile_step(t, c0, s_even, s_odd, std::true_type{});
        tile_step(t + 1, c1, s_odd, s_even, std::true_type{});
      }
    }
    generic_pairs_to(t_end);
    if (t < t_end) tile_step(t, c0, s_even, s_odd, std::false_type{});
  }
#undef AXL_K_FRAG
#undef AXL_S_PLAIN

  // Epilogue: out = acc / l ; lse = m*scale + ln(l).
  const float l_tot = xor32_sum(l_run);
  float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;  // a row with no visible key yields zeros
  if constexpr (AUX) inv_l *= a.aux.keep_scale;
  __bf16* op = (__bf16*)a.out + b * a.os.b + (int64_t)(q0 + l32) * a.os.s + h * a.os.h;
#pragma unroll
  for (int dt = 0; dt < DT; dt++) {
#pragma unroll
    for (int rq = 0; rq < 4; rq++) {
      union {
        bf16x2 p[2];
        uint2 u;
      } w;
      w.p[0] = E::pack(o[dt][4 * rq + 0] * inv_l, o[dt][4 * rq + 1] * inv_l);
      w.p[1] = E::pack(o[dt][4 * rq + 2] * inv_l, o[dt][4 * rq + 3] * inv_l);
      if (32 * dt + 8 * rq + 4 * g < a.d_real) *(uint2*)(op + 32 * dt + 8 * rq + 4 * g) = w.u;
    }
  }
  if (a.lse && g == 0) {
    a.lse[((int64_t)b * a.Hq + h) * a.T + q0 + l32] = (m_run * c + fast_log2(l_tot)) * kLn2;
  }
}

// ---------------------------------------------------------------------------------------------
// fp32 forward: same mapping with v_mfma_f32_32x32x2_f32 (true fp32 multiply-accumulate), K and V
// staged in LDS as fp32; exp via the accurate libm path.  Each wavefront owns 32 query rows and a
// 32-key tile per step.
// ---------------------------------------------------------------------------------------------
template <int D>
struct FwdTileF32 {
  static constexpr int BQ = 128;
  static constexpr int BK = 32;
  static constexpr int KSTRIDE = D * 4 + 4;   // bytes; +1 word: lanes read a column of rows
  static constexpr int VSTRIDE = D * 4;       // lanes read consecutive d of one row: no pad needed
  static constexpr int KBYTES = BK * KSTRIDE;
  static constexpr int VBYTES = BK * VSTRIDE;
  static constexpr int BUF_BYTES = KBYTES + VBYTES;   // one K / V tile; tile t lives in buffer t % 2
  static constexpr int QSTRIDE = D * 4 + 4;
  static constexpr int QBYTES = BQ * QSTRIDE;         // the query block passes through the same memory once
  static constexpr int LDS_BYTES = 2 * BUF_BYTES > QBYTES ? 2 * BUF_BYTES : QBYTES;
  static constexpr int LD4 = BK * (D / 4) / 256;      // float4 loads per thread and tensor tile
  static_assert(BK * (D / 4) % 256 == 0, "a tile divides evenly over the threads");
};

template <int D>
__global__ __launch_bounds__(256) void flash_fwd_f32_kernel(const FwdArgs a) {
  using Tile = FwdTileF32<D>;
  constexpr int DT = D / 32;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* const q_lds = (float*)smem;
  constexpr int QS = Tile::QSTRIDE / 4, KS = Tile::KSTRIDE / 4, VS = Tile::VSTRIDE / 4;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  int qb, b, h;
  // all pairs of an XCD in one group: query blocks in the globally longest-first order
  decode_block(blockIdx.x, a.T / Tile::BQ, a.B, a.Hq, a.Hkv, 1 << 20, qb, b, h);
  const int hk = h / (a.Hq / a.Hkv);
  const int q_off = a.q_off + (a.q_offs ? a.q_offs[b] : 0);  // position of this sequence's query row 0
  const int q0_wg = qb * Tile::BQ;
  const int q0 = q0_wg + wave * 32;

  const float* qg = (const float*)a.q + b * a.qs.b + (int64_t)q0_wg * a.qs.s + h * a.qs.h;
  const float* kp = (const float*)a.k + b * a.ks.b + hk * a.ks.h;
  const float* vp = (const float*)a.v + b * a.vs.b + hk * a.vs.h;

  // The 128 x D query block (fp32) passes through LDS once; a lane keeps the half of its own row that
  // its MFMAs read (elements 2 d2 + g) in registers.
  for (int i = tid; i < Tile::BQ * (D / 4); i += 256) {
    const int row = i / (D / 4), c4 = i % (D / 4);
    const float4 x = *(const float4*)(qg + (int64_t)row * a.qs.s + c4 * 4);
    float* dst = q_lds + row * QS + c4 * 4;
    dst[0] = x.x; dst[1] = x.y; dst[2] = x.z; dst[3] = x.w;
  }
  __syncthreads();
  float q_mine[D / 2];
  {
    const float* q_row = q_lds + (wave * 32 + l32) * QS;
#pragma unroll
    for (int d2 = 0; d2 < D / 2; d2++) q_mine[d2] = q_row[2 * d2 + g];
  }
  __syncthreads();  // the ring of K / V tiles takes the memory over

  int k_begin = 0, k_end = a.S;
  if (a.mask_kind != AXL_MASK_NONE) {
    k_end = min(a.S, q0_wg + Tile::BQ + q_off);
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) k_begin = max(0, q0_wg + q_off - a.window);
  }
  const int t_begin = k_begin / Tile::BK;
  const int t_end = (k_end + Tile::BK - 1) / Tile::BK;
  const int qpos = q0 + l32 + q_off;
  const int qpos_min = q0 + q_off, qpos_max = q0 + 31 + q_off;
  const int seg_q = a.seg ? a.seg[(int64_t)b * a.T + q0 + l32] : 0;
  const int32_t* seg_k = a.seg ? a.seg + (int64_t)b * a.T : nullptr;
  const char* bias_row = nullptr;
  const uint8_t* drop_row = nullptr;
  if (a.aux.bias) bias_row = a.aux.bias + b * a.aux.bias_sb + h * a.aux.bias_sh + (int64_t)(q0 + l32) * a.aux.bias_sr;
  if (a.aux.drop) drop_row = a.aux.drop + b * a.aux.drop_sb + h * a.aux.drop_sh + (int64_t)(q0 + l32) * a.aux.drop_sr;

  floatx16 o[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[i][r] = 0.f;
  float m_run = kNegInf, l_run = 0.f;
  if (a.sink) {  // the sink logit counts as an already-processed key without a value row
    m_run = a.sink[h];
    l_run = g == 0 ? 1.f : 0.f;
  }
  // The K / V tile of 32 keys from global memory into this thread's registers, and from there into a
  // ring buffer: the next tile's round trip runs under the current tile's MFMAs, one barrier per tile.
  float4 kx[Tile::LD4], vx[Tile::LD4];
  auto request = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < Tile::LD4; i++) {
      const int e = tid + i * 256, row = e / (D / 4), c4 = e % (D / 4);
      kx[i] = *(const float4*)(kp + (int64_t)(k0 + row) * a.ks.s + c4 * 4);
      vx[i] = *(const float4*)(vp + (int64_t)(k0 + row) * a.vs.s + c4 * 4);
    }
  };
  auto deposit = [&](int t) __attribute__((always_inline)) {
    float* k_dst = (float*)(smem + (t & 1) * Tile::BUF_BYTES);
    float* v_dst = (float*)(smem + (t & 1) * Tile::BUF_BYTES + Tile::KBYTES);
#pragma unroll
    for (int i = 0; i < Tile::LD4; i++) {
      const int e = tid + i * 256, row = e / (D / 4), c4 = e % (D / 4);
      float* kd = k_dst + row * KS + c4 * 4;
      kd[0] = kx[i].x; kd[1] = kx[i].y; kd[2] = kx[i].z; kd[3] = kx[i].w;
      *(float4*)(v_dst + row * VS + c4 * 4) = vx[i];
    }
  };
  if (t_begin < t_end) {
    request(t_begin * Tile::BK);
    deposit(t_begin);
  }
  __syncthreads();

  for (int t = t_begin; t < t_end; t++) {
    const int k0 = t * Tile::BK;
    const bool more = t + 1 < t_end;
    if (more) request(k0 + Tile::BK);
    const float* k_lds = (const float*)(smem + (t & 1) * Tile::BUF_BYTES);
    const float* v_lds = (const float*)(smem + (t & 1) * Tile::BUF_BYTES + Tile::KBYTES);
    bool skip = false;
    if (a.mask_kind != AXL_MASK_NONE) {
      skip = k0 > qpos_max;
      if (a.mask_kind == AXL_MASK_SLIDING_WINDOW)
        skip = skip || (qpos_min - (k0 + Tile::BK - 1) > a.window);
    }
    if (!skip) {
    // S^T[key][q]: A = K (lane: key row l32, k index g), B = Q^T (lane: query l32, k index g).
    floatx16 s;
#pragma unroll
    for (int r = 0; r < 16; r++) s[r] = 0.f;
    const float* k_row = k_lds + l32 * KS;
#pragma unroll
    for (int d2 = 0; d2 < D / 2; d2++) {
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(k_row[2 * d2 + g], q_mine[d2], s, 0, 0, 0);
    }
    // Register r of lane group g is key k0 + 8(r/4) + 4g + (r%4).
    if (bias_row) {  // logits = scale * qk + bias: pre-divide so the common scale below applies
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++) {
        float bv[4];
        load_bias<4>(bias_row, k0 + 8 * r4 + 4 * g, a.aux.bias_f32, bv);
#pragma unroll
        for (int j = 0; j < 4; j++) s[4 * r4 + j] += bv[j] * a.aux.inv_scale;
      }
    }
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int kpos = k0 + 8 * (r / 4) + 4 * g + (r % 4);
      bool keep = true;
      if (a.mask_kind != AXL_MASK_NONE) {
        const int diff = qpos - kpos;
        keep = diff >= 0;
        if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) keep = keep && diff <= a.window;
      }
      if (seg_k) keep = keep && (seg_k[kpos] == seg_q);
      s[r] = keep ? s[r] * a.scale : kMasked;
    }
    float mx = m_run;
#pragma unroll
    for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[r]);
    mx = xor32_max(mx);
    const float corr = expf(m_run - mx);
    m_run = mx;
    float lsum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      s[r] = expf(s[r] - mx);
      lsum += s[r];
    }
    l_run = l_run * corr + lsum;
    if (drop_row) {  // dropped probabilities leave P V but stay in the row sum
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++) {
        const unsigned w = *(const unsigned*)(drop_row + k0 + 8 * r4 + 4 * g);
#pragma unroll
        for (int j = 0; j < 4; j++) s[4 * r4 + j] = ((w >> (8 * j)) & 0xffu) ? 0.f : s[4 * r4 + j];
      }
    }
#pragma unroll
    for (int i = 0; i < DT; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[i][r] *= corr;
    // O^T[d][q] += V^T[d][key] P^T[key][q]; one key per lane group per MFMA: group g supplies
    // register r, i.e. key 8(r/4) + 4g + (r%4).
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const float* v_row = v_lds + (8 * (r / 4) + 4 * g + (r % 4)) * VS + l32;
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(v_row[32 * dt], s[r], o[dt], 0, 0, 0);
    }
    }  // tile not skipped
    if (more) deposit(t + 1);  // that buffer was last read a tile ago, before the barrier that ended it
    __syncthreads();
  }

  const float l_tot = xor32_sum(l_run);
  const float inv_l = (l_tot > 0.f ? 1.0f / l_tot : 0.f) * a.aux.keep_scale;  // no visible key: zeros
  float* op = (float*)a.out + b * a.os.b + (int64_t)(q0 + l32) * a.os.s + h * a.os.h;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int rq = 0; rq < 4; rq++) {
      float4 w = {o[dt][4 * rq + 0] * inv_l, o[dt][4 * rq + 1] * inv_l, o[dt][4 * rq + 2] * inv_l,
                  o[dt][4 * rq + 3] * inv_l};
      *(float4*)(op + 32 * dt + 8 * rq + 4 * g) = w;
    }
  if (a.lse && g == 0) a.lse[((int64_t)b * a.Hq + h) * a.T + q0 + l32] = m_run + logf(l_tot);
}

// ---------------------------------------------------------------------------------------------
// fp32 forward on the 16-bit matrix instruction.  This GPU multiplies bf16 sixteen times as fast as
// fp32 (v_mfma_f32_32x32x16_bf16 against v_mfma_f32_32x32x2_f32), so an fp32 operand travels as three
// bf16 values, x = hi + mid + lo (8 + 8 + 8 bits of significand, each the rounded remainder of the one
// before: the split is exact), and a product of two operands as the six partial products that matter,
//   a b ~ a_lo b_hi + a_hi b_lo + a_mid b_mid + a_mid b_hi + a_hi b_mid + a_hi b_hi,
// accumulated in fp32 by the instruction; the three products left out are below 2^-24 of the result.
// Measured against float64 the error is that of an fp32 dot product (or smaller: fewer roundings).
// Six 32-cycle instructions per 16 elements of the inner dimension instead of eight 64-cycle ones.
//
// Mapping as in the kernel above (a wavefront owns 32 query rows, a 32-key tile per step, S^T and O^T
// accumulators with the query as the lane's column), operand layouts as in the 16-bit kernel: K rows
// are read in the order swap_bits_2_3, so that registers 0..7 / 8..15 of a lane's S^T column are the
// keys 8g .. 8g+7 of the tile's first / second half and, split and packed, are the B operand of
// O^T += V^T P^T as they stand; V^T comes out of transposing LDS reads.  K and V tiles go from global
// memory through registers, where they are split, into three 16-bit planes each in LDS.
// ---------------------------------------------------------------------------------------------
template <int D, int NW>
struct FwdTileF32x {
  static constexpr int NT = 64 * NW;          // threads: NW wavefronts of 32 query rows
  static constexpr int BQ = 32 * NW;
  static constexpr int BK = 32;
  static constexpr int KSTRIDE = D * 2 + 16;  // bytes per key row of a plane: 16 rows read by 16 lanes hit all banks
  static constexpr int VSTRIDE = D * 2 + 64;  // the same for the 4 rows x 2 halves of a transposing read
  static constexpr int KPLANE = BK * KSTRIDE, VPLANE = BK * VSTRIDE;
  static constexpr int BUF_BYTES = 3 * (KPLANE + VPLANE);   // one K / V tile; tile t lives in buffer t % 2
  static constexpr int QSTRIDE = D * 4 + 4;
  static constexpr int QBYTES = BQ * QSTRIDE;               // the query block passes through the same memory once
  static constexpr int LDS_BYTES = 2 * BUF_BYTES > QBYTES ? 2 * BUF_BYTES : QBYTES;
  static constexpr int LD4 = BK * (D / 4) / NT;             // float4 loads per thread and tensor tile
  static_assert(BK * (D / 4) % NT == 0, "a tile divides evenly over the threads");
};

template <int D, int NW>
__global__ __launch_bounds__(64 * NW) void flash_fwd_f32x_kernel(const FwdArgs a) {
  using Tile = FwdTileF32x<D, NW>;
  constexpr int DT = D / 32, KSTEPS = D / 16;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* const q_lds = (float*)smem;
  constexpr int QS = Tile::QSTRIDE / 4;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  int qb, b, h;
  decode_block(blockIdx.x, a.T / Tile::BQ, a.B, a.Hq, a.Hkv, 1 << 20, qb, b, h);
  const int hk = h / (a.Hq / a.Hkv);
  const int q_off = a.q_off + (a.q_offs ? a.q_offs[b] : 0);  // position of this sequence's query row 0
  const int q0_wg = qb * Tile::BQ;
  const int q0 = q0_wg + wave * 32;

  const float* qg = (const float*)a.q + b * a.qs.b + (int64_t)q0_wg * a.qs.s + h * a.qs.h;
  const float* kp = (const float*)a.k + b * a.ks.b + hk * a.ks.h;
  const float* vp = (const float*)a.v + b * a.vs.b + hk * a.vs.h;

  // The 128 x D query block passes through LDS once; a lane keeps, split, the half of its own row that its
  // MFMAs read (elements 16 s + 8 g .. + 7 of every 16).
  for (int i = tid; i < Tile::BQ * (D / 4); i += Tile::NT) {
    const int row = i / (D / 4), c4 = i % (D / 4);
    const float4 x = *(const float4*)(qg + (int64_t)row * a.qs.s + c4 * 4);
    float* dst = q_lds + row * QS + c4 * 4;
    dst[0] = x.x; dst[1] = x.y; dst[2] = x.z; dst[3] = x.w;
  }
  __syncthreads();
  // Logits are kept in units of log2: Q is multiplied by scale * log2(e) ahead of its split, the
  // exponentials are exp2 (v_exp_f32, 1 ulp), and lse is converted back at the end.
  const float c = a.scale * kLog2e;
  bf16x8 q_mine[KSTEPS][3];
  {
    const float* q_row = q_lds + (wave * 32 + l32) * QS;
#pragma unroll
    for (int s = 0; s < KSTEPS; s++) {
      float x[8];
#pragma unroll
      for (int j = 0; j < 8; j++) x[j] = q_row[16 * s + 8 * g + j] * c;
      Split3x8 sp;
      split3x8(x, sp);
#pragma unroll
      for (int p = 0; p < 3; p++) q_mine[s][p] = sp.part[p].v;
    }
  }
  __syncthreads();  // the ring of K / V tiles takes the memory over

  int k_begin = 0, k_end = a.S;
  if (a.mask_kind != AXL_MASK_NONE) {
    k_end = min(a.S, q0_wg + Tile::BQ + q_off);
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) k_begin = max(0, q0_wg + q_off - a.window);
  }
  const int t_begin = k_begin / Tile::BK;
  const int t_end = (k_end + Tile::BK - 1) / Tile::BK;
  const int qpos = q0 + l32 + q_off;
  const int qpos_min = q0 + q_off, qpos_max = q0 + 31 + q_off;
  const int seg_q = a.seg ? a.seg[(int64_t)b * a.T + q0 + l32] : 0;
  const int32_t* seg_k = a.seg ? a.seg + (int64_t)b * a.T : nullptr;
  const char* bias_row = nullptr;
  const uint8_t* drop_row = nullptr;
  if (a.aux.bias) bias_row = a.aux.bias + b * a.aux.bias_sb + h * a.aux.bias_sh + (int64_t)(q0 + l32) * a.aux.bias_sr;
  if (a.aux.drop) drop_row = a.aux.drop + b * a.aux.drop_sb + h * a.aux.drop_sh + (int64_t)(q0 + l32) * a.aux.drop_sr;

  floatx16 o[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[i][r] = 0.f;
  float m_run = kNegInf, l_run = 0.f;
  if (a.sink) {  // the sink logit counts as an already-processed key without a value row
    m_run = a.sink[h] * kLog2e;
    l_run = g == 0 ? 1.f : 0.f;
  }
  // The K / V tile of 32 keys from global memory into this thread's registers, and from there, split, into
  // a ring buffer: the next tile's round trip runs under the current tile's MFMAs, one barrier per tile.
  float4 kx[Tile::LD4], vx[Tile::LD4];
  auto request = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < Tile::LD4; i++) {
      const int e = tid + i * Tile::NT, row = e / (D / 4), c4 = e % (D / 4);
      kx[i] = *(const float4*)(kp + (int64_t)(k0 + row) * a.ks.s + c4 * 4);
      vx[i] = *(const float4*)(vp + (int64_t)(k0 + row) * a.vs.s + c4 * 4);
    }
  };
  auto deposit = [&](int t) __attribute__((always_inline)) {
    char* k_dst = smem + (t & 1) * Tile::BUF_BYTES;
    char* v_dst = k_dst + 3 * Tile::KPLANE;
#pragma unroll
    for (int i = 0; i < Tile::LD4; i++) {
      const int e = tid + i * Tile::NT, row = e / (D / 4), c4 = e % (D / 4);
      const Split3x2 k01 = split3(kx[i].x, kx[i].y), k23 = split3(kx[i].z, kx[i].w);
      const Split3x2 v01 = split3(vx[i].x, vx[i].y), v23 = split3(vx[i].z, vx[i].w);
#pragma unroll
      for (int p = 0; p < 3; p++) {
        union { bf16x2 h[2]; uint2 u; } kw, vw;
        kw.h[0] = k01.part[p]; kw.h[1] = k23.part[p];
        vw.h[0] = v01.part[p]; vw.h[1] = v23.part[p];
        *(uint2*)(k_dst + p * Tile::KPLANE + row * Tile::KSTRIDE + c4 * 8) = kw.u;
        *(uint2*)(v_dst + p * Tile::VPLANE + row * Tile::VSTRIDE + c4 * 8) = vw.u;
      }
    }
  };
  if (t_begin < t_end) {
    request(t_begin * Tile::BK);
    deposit(t_begin);
  }
  __syncthreads();

  // Per-lane read offsets.  K: the row of key swap_bits_2_3(l32), 16 bytes at d = 16 s + 8 g.  V: transposing
  // reads at row 8 g + j16 / 4 (+4 for the second half, +16 for the tile's second 16 keys), columns
  // 32 dt + 16 half + 4 (j16 % 4) .. + 3.
  const int k_off = swap_bits_2_3(l32) * Tile::KSTRIDE + 16 * g;
  const int j16 = lane & 15, half = (lane >> 4) & 1;
  const int v_off = (8 * g + (j16 >> 2)) * Tile::VSTRIDE + (16 * half + 4 * (j16 & 3)) * 2;

  for (int t = t_begin; t < t_end; t++) {
    const int k0 = t * Tile::BK;
    const bool more = t + 1 < t_end;
    if (more) request(k0 + Tile::BK);
    const char* k_lds = smem + (t & 1) * Tile::BUF_BYTES;
    const char* v_lds = k_lds + 3 * Tile::KPLANE;
    bool skip = false;
    if (a.mask_kind != AXL_MASK_NONE) {
      skip = k0 > qpos_max;
      if (a.mask_kind == AXL_MASK_SLIDING_WINDOW)
        skip = skip || (qpos_min - (k0 + Tile::BK - 1) > a.window);
    }
    if (!skip) {
    // S^T[key][q]: A = K rows, B = Q^T.
    floatx16 s;
#pragma unroll
    for (int r = 0; r < 16; r++) s[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      bf16x8 kf[3];
#pragma unroll
      for (int p = 0; p < 3; p++) kf[p] = *(const bf16x8*)(k_lds + p * Tile::KPLANE + k_off + 32 * ks);
      s = mfma_split(kf, q_mine[ks], s);
    }
    // Register r of lane group g is key k0 + 16 (r / 8) + 8 g + r % 8.
    if (bias_row) {  // logits = scale * qk + bias, in units of log2
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++) {
        float bv[4];
        load_bias<4>(bias_row, k0 + 16 * (r4 / 2) + 8 * g + 4 * (r4 % 2), a.aux.bias_f32, bv);
#pragma unroll
        for (int j = 0; j < 4; j++) s[4 * r4 + j] += bv[j] * kLog2e;
      }
    }
    // A tile in the interior of the wavefront's range (every key at or before its first query and inside
    // the window of its last one, no segment ids) has nothing to mask.
    bool interior = seg_k == nullptr;
    if (a.mask_kind != AXL_MASK_NONE) {
      interior = interior && k0 + Tile::BK - 1 <= qpos_min;
      if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) interior = interior && qpos_max - k0 <= a.window;
    }
    if (!interior) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int kpos = k0 + 16 * (r / 8) + 8 * g + (r % 8);
        bool keep = true;
        if (a.mask_kind != AXL_MASK_NONE) {
          const int diff = qpos - kpos;
          keep = diff >= 0;
          if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) keep = keep && diff <= a.window;
        }
        if (seg_k) keep = keep && (seg_k[kpos] == seg_q);
        s[r] = keep ? s[r] : kMasked;
      }
    }
    float mx = m_run;
#pragma unroll
    for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[r]);
    mx = xor32_max(mx);
    // The running maximum moves in the first few tiles of a row and rarely after: the rescaling is left
    // out (its factor would be exactly 1) unless it moved for some row of the wavefront.
    const bool moved = __builtin_amdgcn_ballot_w64(mx != m_run) != 0;
    if (moved) {
      const float corr = fast_exp2(m_run - mx);
      l_run *= corr;
#pragma unroll
      for (int i = 0; i < DT; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[i][r] *= corr;
    }
    m_run = mx;
    float lsum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      s[r] = fast_exp2(s[r] - mx);
      lsum += s[r];
    }
    l_run += lsum;
    if (drop_row) {  // dropped probabilities leave P V but stay in the row sum
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++) {
        const unsigned w = *(const unsigned*)(drop_row + k0 + 16 * (r4 / 2) + 8 * g + 4 * (r4 % 2));
#pragma unroll
        for (int j = 0; j < 4; j++) s[4 * r4 + j] = ((w >> (8 * j)) & 0xffu) ? 0.f : s[4 * r4 + j];
      }
    }
    // O^T[d][q] += V^T[d][key] P^T[key][q], 16 keys per step.
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
      float pr[8];
#pragma unroll
      for (int j = 0; j < 8; j++) pr[j] = s[8 * kk + j];
      Split3x8 ps;
      split3x8(pr, ps);
      const bf16x8 pf[3] = {ps.part[0].v, ps.part[1].v, ps.part[2].v};
#pragma unroll
      for (int dt = 0; dt < DT; dt++) {
        union { bf16x8 v; shortx4 hlf[2]; } vf[3];
#pragma unroll
        for (int p = 0; p < 3; p++) {
          const char* va = v_lds + p * Tile::VPLANE + v_off + 16 * kk * Tile::VSTRIDE + 64 * dt;
          vf[p].hlf[0] = lds_read_tr16(va);
          vf[p].hlf[1] = lds_read_tr16(va + 4 * Tile::VSTRIDE);
        }
        const bf16x8 vfa[3] = {vf[0].v, vf[1].v, vf[2].v};
        o[dt] = mfma_split(vfa, pf, o[dt]);
      }
    }
    }  // tile not skipped
    if (more) deposit(t + 1);  // that buffer was last read a tile ago, before the barrier that ended it
    __syncthreads();
  }

  const float l_tot = xor32_sum(l_run);
  const float inv_l = (l_tot > 0.f ? 1.0f / l_tot : 0.f) * a.aux.keep_scale;  // no visible key: zeros
  float* op = (float*)a.out + b * a.os.b + (int64_t)(q0 + l32) * a.os.s + h * a.os.h;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int rq = 0; rq < 4; rq++) {
      float4 w = {o[dt][4 * rq + 0] * inv_l, o[dt][4 * rq + 1] * inv_l, o[dt][4 * rq + 2] * inv_l,
                  o[dt][4 * rq + 3] * inv_l};
      *(float4*)(op + 32 * dt + 8 * rq + 4 * g) = w;
    }
  if (a.lse && g == 0) a.lse[((int64_t)b * a.Hq + h) * a.T + q0 + l32] = m_run * kLn2 + logf(l_tot);
}

static Strides3 to_s3(const AxlStrides& s) { return Strides3{s.batch, s.seq, s.head}; }

int launch_flash_fwd(const AxlFlashFwdParams& p, hipStream_t stream) {
  FwdArgs a;
  a.q = p.q; a.k = p.k; a.v = p.v; a.out = p.out; a.lse = p.lse; a.seg = p.segment_ids;
  a.sink = p.logit_sink;
  a.aux = make_aux_args(p.aux, p.softmax_scale);
  const bool aux = p.aux.bias || p.aux.dropout_mask;
  a.qs = to_s3(p.q_strides); a.ks = to_s3(p.k_strides); a.vs = to_s3(p.v_strides);
  a.os = to_s3(p.out_strides);
  a.B = p.batch; a.T = p.q_len; a.S = p.kv_len; a.Hq = p.num_q_heads; a.Hkv = p.num_kv_heads;
  a.mask_kind = p.mask_kind; a.window = p.sliding_window; a.q_off = p.q_pos_offset;
  a.q_offs = p.q_pos_offsets;
  a.scale = p.softmax_scale;
  a.d_real = p.head_dim;
  const int width = p.head_dim <= 64 ? 64 : 128;  // the compiled width that serves this head_dim
  hipError_t err = hipSuccess;
#define AXL_LAUNCH_FWD(KERNEL, TILE)                                                            \
  do {                                                                                          \
    err = allow_dynamic_lds((const void*)KERNEL, TILE::LDS_BYTES);                              \
    if (err == hipSuccess) {                                                                    \
      const int grid = (p.q_len / TILE::BQ) * p.batch * p.num_q_heads;                          \
      hipLaunchKernelGGL(KERNEL, dim3(grid), dim3(2 * TILE::BQ), TILE::LDS_BYTES, stream, a);   \
      err = hipGetLastError();                                                                  \
    }                                                                                           \
  } while (0)
#define AXL_LAUNCH_FWD16(E)                                                                     \
  do {                                                                                          \
    if (width == 128) {                                                                         \
      if (aux) AXL_LAUNCH_FWD((flash_fwd_kernel<E, 128, true>), FwdTile<128>);                  \
      else AXL_LAUNCH_FWD((flash_fwd_kernel<E, 128, false>), FwdTile<128>);                     \
    } else {                                                                                    \
      if (aux) AXL_LAUNCH_FWD((flash_fwd_kernel<E, 64, true>), FwdTile<64>);                    \
      else AXL_LAUNCH_FWD((flash_fwd_kernel<E, 64, false>), FwdTile<64>);                       \
    }                                                                                           \
  } while (0)
  if (p.dtype == AXL_BF16) {
    AXL_LAUNCH_FWD16(ElemBf16);
  } else if (p.dtype == AXL_F16) {
    AXL_LAUNCH_FWD16(ElemF16);
  } else {
    // AXL_F32_MFMA=1 in the environment: the kernel on the fp32 matrix instruction (for comparison).
    static const bool true_f32 = [] { const char* e = getenv("AXL_F32_MFMA"); return e && e[0] == '1'; }();
    if (true_f32) {
      if (p.head_dim == 128) AXL_LAUNCH_FWD(flash_fwd_f32_kernel<128>, FwdTileF32<128>);
      else AXL_LAUNCH_FWD(flash_fwd_f32_kernel<64>, FwdTileF32<64>);
    } else {
      // eight wavefronts (two per SIMD, 256 query rows share a tile's split) where the length allows and such
      // workgroups are still at least as many as the CUs (a small call is bound by its longest workgroup)
      static const bool four = [] { const char* e = getenv("AXL_F32X_WAVES"); return e && e[0] == '4'; }();
      using T128x8 = FwdTileF32x<128, 8>;
      using T64x8 = FwdTileF32x<64, 8>;
      using T128x4 = FwdTileF32x<128, 4>;
      using T64x4 = FwdTileF32x<64, 4>;
      if (p.q_len % 256 == 0 && !four && (int64_t)(p.q_len / 256) * p.batch * p.num_q_heads >= cu_count()) {
        if (p.head_dim == 128) AXL_LAUNCH_FWD((flash_fwd_f32x_kernel<128, 8>), T128x8);
        else AXL_LAUNCH_FWD((flash_fwd_f32x_kernel<64, 8>), T64x8);
      } else {
        if (p.head_dim == 128) AXL_LAUNCH_FWD((flash_fwd_f32x_kernel<128, 4>), T128x4);
        else AXL_LAUNCH_FWD((flash_fwd_f32x_kernel<64, 4>), T64x4);
      }
    }
  }
#undef AXL_LAUNCH_FWD16
#undef AXL_LAUNCH_FWD
  if (err != hipSuccess)
    return set_error(AXL_ERR_LAUNCH, "axl_flash_fwd: launch failed: %s", hipGetErrorString(err));
  return AXL_OK;
}

}  // namespace axl
