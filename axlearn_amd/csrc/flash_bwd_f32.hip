// fp32 flash-attention backward for gfx950: dQ and dK/dV.  Two pairs of kernels: the first with
// v_mfma_f32_32x32x2_f32 (fp32 multiply-accumulate) and the accurate exponential, kept for comparison
// (AXL_F32_MFMA=1 in the environment); the second, which runs by default, with every fp32 product formed
// from bf16 parts on v_mfma_f32_32x32x16_bf16 (second half of this file), to the same accuracy.
//
// Replaces the float32 case of axlearn/common/flash_attention/gpu_attention.py:621-786
// (`_mha_backward`, which shrinks its blocks to 32 for float32 inputs, :645-646, and whose tests run
// float32 forward + backward, gpu_attention_test.py:197) with
//   p  = exp(scale * q k^T + bias - lse)                    (:507, :599)
//   dp = dO v^T, zeroed where dropped and scaled by 1/(1-rate)   (:508-512, :600-603)
//   ds = p * (dp - delta)                                   (:514, :604)
//   dv += (p after dropout)^T dO,  dk += scale * ds^T q,  dq += scale * ds k   (:513, :518, :608)
//
// A workgroup of 4 wavefronts owns 128 rows (queries in the dQ kernel, keys in the dK/dV kernel), 32
// per wavefront, one wavefront per SIMD.  A lane keeps the half of its own row that its MFMAs read
// (elements 2 d2 + g of the row: the fp32 matrix instruction takes one element per lane and step) in
// registers for the whole kernel, next to the fp32 accumulators (the dK/dV kernel, whose two accumulator
// sets leave less room, keeps its V rows in LDS instead); the 32-row tiles it loops over come
// through a double-buffered LDS copy whose next tile is on its way from global memory while the
// current one is multiplied, with one barrier per tile.  The mapping is the forward's (flash_fwd.hip,
// fp32 kernel): an accumulator register r of lane (l32, g) is row 8(r/4) + 4g + (r%4), column l32, so
// a product whose reduction runs over the accumulator's rows takes register r itself as the B operand
// of MFMA r ("one reduction index per lane group per MFMA").
#include <cstdlib>

#include "flash_bwd.h"

namespace axl {

template <int D>
struct BwdTileF32 {
  static constexpr int NT = 256;               // threads of a workgroup
  static constexpr int ROWS = 128;             // rows owned by a workgroup (4 wavefronts x 32)
  static constexpr int TILE = 32;              // rows of the tiles it loops over
  static constexpr int PS = D + 1;             // words per LDS row: lanes read a column of rows
  static constexpr int TILE_WORDS = TILE * PS;
  static constexpr int BUF_WORDS = 2 * TILE_WORDS + 2 * TILE;   // two tensors' tiles, two rows of statistics
  static constexpr int LDS_BYTES = 2 * BUF_WORDS * 4;
  static constexpr int OWN_WORDS = ROWS * PS;                   // one owned tensor kept in LDS (dK/dV kernel: V)
  static constexpr int LDS_BYTES_DKDV = LDS_BYTES + OWN_WORDS * 4;
  static constexpr int LD4 = TILE * (D / 4) / NT;               // float4 loads per thread and tensor tile
  static_assert(TILE * (D / 4) % NT == 0, "a tile divides evenly over the threads");
  static_assert(4 * TILE_WORDS <= 2 * BUF_WORDS, "the owned rows pass through the ring, 128 at a time");
};

__device__ __forceinline__ float bias_at(const AuxArgs& x, const char* row, int col) {
  if (x.bias_f32) return *(const float*)(row + (int64_t)col * 4);
  return (float)*(const __bf16*)(row + (int64_t)col * 2);
}

// The 32 x D tile at `src` (row stride `stride` elements) into this thread's registers, and from there
// into LDS rows of PS words.
template <int D>
__device__ __forceinline__ void tile_request(float4 (&x)[BwdTileF32<D>::LD4], const float* src, int64_t stride, int tid) {
  using Tile = BwdTileF32<D>;
#pragma unroll
  for (int i = 0; i < Tile::LD4; i++) {
    const int e = tid + i * Tile::NT, row = e / (D / 4), c4 = e % (D / 4);
    x[i] = *(const float4*)(src + (int64_t)row * stride + c4 * 4);
  }
}
template <int D>
__device__ __forceinline__ void tile_deposit(float* lds, const float4 (&x)[BwdTileF32<D>::LD4], int tid) {
  using Tile = BwdTileF32<D>;
#pragma unroll
  for (int i = 0; i < Tile::LD4; i++) {
    const int e = tid + i * Tile::NT, row = e / (D / 4), c4 = e % (D / 4);
    float* dst = lds + row * Tile::PS + c4 * 4;
    dst[0] = x[i].x; dst[1] = x[i].y; dst[2] = x[i].z; dst[3] = x[i].w;
  }
}

// The workgroup's 128 owned rows of one tensor pass through LDS once (`lds`: 128 rows of PS words) and
// every lane keeps elements 2 d2 + g of its row.  Called by all threads; contains barriers.
template <int D>
__device__ __forceinline__ void own_rows(float (&mine)[D / 2], float* lds, const float* src, int64_t stride, int tid) {
  using Tile = BwdTileF32<D>;
  __syncthreads();  // whoever read this memory before is done
  for (int i = tid; i < Tile::ROWS * (D / 4); i += Tile::NT) {
    const int row = i / (D / 4), c4 = i % (D / 4);
    const float4 x = *(const float4*)(src + (int64_t)row * stride + c4 * 4);
    float* dst = lds + row * Tile::PS + c4 * 4;
    dst[0] = x.x; dst[1] = x.y; dst[2] = x.z; dst[3] = x.w;
  }
  __syncthreads();
  const int lane = tid & 63, g = lane >> 5;
  const float* row = lds + ((tid >> 6) * 32 + (lane & 31)) * Tile::PS;
#pragma unroll
  for (int d2 = 0; d2 < D / 2; d2++) mine[d2] = row[2 * d2 + g];
}

// ---------------------------------------------------------------------------------------------
// dQ: a workgroup owns 128 query rows of one head and loops over 32-key tiles.
//   S^T[key][q] = K Q^T and dP^T[key][q] = V dO^T (A = K / V row l32, B = Q / dO row l32), so lane
//   (l32, g) holds query l32 and keys 8(r/4) + 4g + (r%4); dQ^T[d][q] += K^T[d][key] dS^T[key][q].
// ---------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void flash_bwd_dq_f32_kernel(const BwdArgs a) {
  using Tile = BwdTileF32<D>;
  constexpr int DT = D / 32, PS = Tile::PS;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* const ring = (float*)smem;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  const int nqb = a.T / Tile::ROWS;
  const int qb = nqb - 1 - blockIdx.x % nqb;  // heaviest blocks of a causal mask first
  const int h = (blockIdx.x / nqb) % a.Hq, b = blockIdx.x / (nqb * a.Hq);
  const int hk = h / (a.Hq / a.Hkv);
  const int q0_wg = qb * Tile::ROWS, q0 = q0_wg + wave * 32;

  float q_mine[D / 2], do_mine[D / 2];
  own_rows<D>(q_mine, ring, (const float*)a.q + b * a.qs.b + (int64_t)q0_wg * a.qs.s + h * a.qs.h, a.qs.s, tid);
  own_rows<D>(do_mine, ring, (const float*)a.dout + b * a.dos.b + (int64_t)q0_wg * a.dos.s + h * a.dos.h, a.dos.s, tid);
  const float* kp = (const float*)a.k + b * a.ks.b + hk * a.ks.h;
  const float* vp = (const float*)a.v + b * a.vs.b + hk * a.vs.h;
  const int64_t stat = ((int64_t)b * a.Hq + h) * a.T + q0 + l32;
  const float lse_q = a.lse[stat], delta_q = -a.ndelta[stat];

  int k_begin = 0, k_end = a.S;
  if (a.mask_kind != AXL_MASK_NONE) {
    k_end = min(a.S, q0_wg + Tile::ROWS + a.q_off);
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) k_begin = max(0, q0_wg + a.q_off - a.window);
  }
  const int t_begin = k_begin / Tile::TILE;
  const int t_end = (k_end + Tile::TILE - 1) / Tile::TILE;
  const int qpos = q0 + l32 + a.q_off;
  const int qpos_min = q0 + a.q_off, qpos_max = q0 + 31 + a.q_off;
  const int seg_q = a.seg ? a.seg[(int64_t)b * a.T + q0 + l32] : 0;
  const int32_t* seg_k = a.seg ? a.seg + (int64_t)b * a.T : nullptr;
  const char* bias_row = nullptr;
  const uint8_t* drop_row = nullptr;
  if (a.aux.bias) bias_row = a.aux.bias + b * a.aux.bias_sb + h * a.aux.bias_sh + (int64_t)(q0 + l32) * a.aux.bias_sr;
  if (a.aux.drop) drop_row = a.aux.drop + b * a.aux.drop_sb + h * a.aux.drop_sh + (int64_t)(q0 + l32) * a.aux.drop_sr;

  floatx16 dq[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq[i][r] = 0.f;

  // Tile t lives in ring buffer t % 2: K rows, then V rows.
  float4 kx[Tile::LD4], vx[Tile::LD4];
  __syncthreads();  // the owned rows have been read out of the ring
  if (t_begin < t_end) {
    tile_request<D>(kx, kp + (int64_t)t_begin * Tile::TILE * a.ks.s, a.ks.s, tid);
    tile_request<D>(vx, vp + (int64_t)t_begin * Tile::TILE * a.vs.s, a.vs.s, tid);
    float* buf = ring + (t_begin & 1) * Tile::BUF_WORDS;
    tile_deposit<D>(buf, kx, tid);
    tile_deposit<D>(buf + Tile::TILE_WORDS, vx, tid);
  }
  __syncthreads();
  for (int t = t_begin; t < t_end; t++) {
    const int k0 = t * Tile::TILE;
    const bool more = t + 1 < t_end;
    if (more) {  // the next tile's round trip runs under this tile's MFMAs
      tile_request<D>(kx, kp + (int64_t)(k0 + Tile::TILE) * a.ks.s, a.ks.s, tid);
      tile_request<D>(vx, vp + (int64_t)(k0 + Tile::TILE) * a.vs.s, a.vs.s, tid);
    }
    const float* k_lds = ring + (t & 1) * Tile::BUF_WORDS;
    const float* v_lds = k_lds + Tile::TILE_WORDS;
    bool skip = false;
    if (a.mask_kind != AXL_MASK_NONE) {
      skip = k0 > qpos_max;
      if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) skip = skip || (qpos_min - (k0 + Tile::TILE - 1) > a.window);
    }
    if (!skip) {
      floatx16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
      const float* k_row = k_lds + l32 * PS;
      const float* v_row = v_lds + l32 * PS;
#pragma unroll
      for (int d2 = 0; d2 < D / 2; d2++) {
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(k_row[2 * d2 + g], q_mine[d2], s, 0, 0, 0);
        dp = __builtin_amdgcn_mfma_f32_32x32x2f32(v_row[2 * d2 + g], do_mine[d2], dp, 0, 0, 0);
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
        float logit = s[r] * a.scale;
        if (bias_row) logit += bias_at(a.aux, bias_row, kpos);
        const float p = keep ? expf(logit - lse_q) : 0.f;
        float dpe = dp[r];
        if (drop_row) dpe = drop_row[kpos] ? 0.f : dpe * a.aux.keep_scale;
        s[r] = p * (dpe - delta_q);  // dS^T
      }
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float* k_col = k_lds + (8 * (r / 4) + 4 * g + (r % 4)) * PS + l32;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
          dq[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(k_col[32 * dt], s[r], dq[dt], 0, 0, 0);
      }
    }
    if (more) {  // the other buffer was last read a tile ago, before the barrier that ended that tile
      float* buf = ring + ((t + 1) & 1) * Tile::BUF_WORDS;
      tile_deposit<D>(buf, kx, tid);
      tile_deposit<D>(buf + Tile::TILE_WORDS, vx, tid);
    }
    __syncthreads();
  }

  float* dqp = (float*)a.dq + b * a.dqs.b + (int64_t)(q0 + l32) * a.dqs.s + h * a.dqs.h;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int rq = 0; rq < 4; rq++) {
      float4 w = {dq[dt][4 * rq + 0] * a.scale, dq[dt][4 * rq + 1] * a.scale, dq[dt][4 * rq + 2] * a.scale,
                  dq[dt][4 * rq + 3] * a.scale};
      *(float4*)(dqp + 32 * dt + 8 * rq + 4 * g) = w;
    }
}

// ---------------------------------------------------------------------------------------------
// dK/dV: a workgroup owns 128 keys of one kv head and loops over the query heads of its group and
// over 32-query tiles.
//   S[q][key] = Q K^T and dP[q][key] = dO V^T (A = Q / dO row l32 of the tile, B = K / V row l32), so
//   lane (l32, g) holds key l32 and queries 8(r/4) + 4g + (r%4);
//   dV^T[d][key] += dO^T[d][q] P[q][key],  dK^T[d][key] += Q^T[d][q] dS[q][key].
// ---------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void flash_bwd_dkdv_f32_kernel(const BwdArgs a) {
  using Tile = BwdTileF32<D>;
  constexpr int DT = D / 32, PS = Tile::PS;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* const ring = (float*)smem;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  const int nkb = a.S / Tile::ROWS;
  const int kb = blockIdx.x % nkb;
  const int hk = (blockIdx.x / nkb) % a.Hkv, b = blockIdx.x / (nkb * a.Hkv);
  const int G = a.Hq / a.Hkv;
  const int k0_wg = kb * Tile::ROWS, k0 = k0_wg + wave * 32;
  const int kpos = k0 + l32;

  float k_mine[D / 2];
  own_rows<D>(k_mine, ring, (const float*)a.k + b * a.ks.b + (int64_t)k0_wg * a.ks.s + hk * a.ks.h, a.ks.s, tid);
  float* const v_own = ring + 2 * Tile::BUF_WORDS;   // the 128 owned V rows stay in LDS
  {
    const float* src = (const float*)a.v + b * a.vs.b + (int64_t)k0_wg * a.vs.s + hk * a.vs.h;
    for (int i = tid; i < Tile::ROWS * (D / 4); i += Tile::NT) {
      const int row = i / (D / 4), c4 = i % (D / 4);
      const float4 x = *(const float4*)(src + (int64_t)row * a.vs.s + c4 * 4);
      float* dst = v_own + row * PS + c4 * 4;
      dst[0] = x.x; dst[1] = x.y; dst[2] = x.z; dst[3] = x.w;
    }
  }
  const float* v_row = v_own + (wave * 32 + l32) * PS;

  // Query rows that can see a key of this block: qpos >= first key, qpos <= last key + window.
  int q_begin = 0, q_end = a.T;
  if (a.mask_kind != AXL_MASK_NONE) {
    q_begin = min(a.T, max(0, k0_wg - a.q_off));
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW)
      q_end = max(q_begin, (int)min((int64_t)a.T, (int64_t)k0_wg + Tile::ROWS + a.window - a.q_off));
  }
  const int t_begin = q_begin / Tile::TILE;
  const int t_end = (q_end + Tile::TILE - 1) / Tile::TILE;
  const int nt = max(t_end - t_begin, 0);
  const int seg_k = a.seg ? a.seg[(int64_t)b * a.T + kpos] : 0;
  const int32_t* seg_q = a.seg ? a.seg + (int64_t)b * a.T : nullptr;

  floatx16 dk[DT], dv[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dk[i][r] = dv[i][r] = 0.f;

  // Step e of the loop is query tile t_begin + e % nt of query head hk G + e / nt; it lives in ring
  // buffer e % 2: Q rows, dO rows, lse and delta of the 32 queries.
  const int steps = nt * G;
  float4 qx[Tile::LD4], dox[Tile::LD4];
  float stat_x = 0.f;  // threads 0..31: lse, 32..63: delta of query tid % 32
  auto request = [&](int e) __attribute__((always_inline)) {
    const int h = hk * G + e / nt, qt0 = (t_begin + e % nt) * Tile::TILE;
    tile_request<D>(qx, (const float*)a.q + b * a.qs.b + h * a.qs.h + (int64_t)qt0 * a.qs.s, a.qs.s, tid);
    tile_request<D>(dox, (const float*)a.dout + b * a.dos.b + h * a.dos.h + (int64_t)qt0 * a.dos.s, a.dos.s, tid);
    const int64_t row = ((int64_t)b * a.Hq + h) * a.T + qt0 + (tid & 31);
    if (tid < 32) stat_x = a.lse[row];
    else if (tid < 64) stat_x = -a.ndelta[row];
  };
  auto deposit = [&](int e) __attribute__((always_inline)) {
    float* buf = ring + (e & 1) * Tile::BUF_WORDS;
    tile_deposit<D>(buf, qx, tid);
    tile_deposit<D>(buf + Tile::TILE_WORDS, dox, tid);
    if (tid < 64) buf[2 * Tile::TILE_WORDS + tid] = stat_x;
  };
  __syncthreads();  // the owned rows have been read out of the ring
  if (steps > 0) {
    request(0);
    deposit(0);
  }
  __syncthreads();
  for (int e = 0; e < steps; e++) {
    const int h = hk * G + e / nt, qt0 = (t_begin + e % nt) * Tile::TILE;
    const bool more = e + 1 < steps;
    if (more) request(e + 1);  // the next tile's round trip runs under this tile's MFMAs
    const float* q_lds = ring + (e & 1) * Tile::BUF_WORDS;
    const float* do_lds = q_lds + Tile::TILE_WORDS;
    const float* lse_lds = q_lds + 2 * Tile::TILE_WORDS;
    const float* delta_lds = lse_lds + Tile::TILE;
    bool skip = false;
    if (a.mask_kind != AXL_MASK_NONE) {
      skip = qt0 + 31 + a.q_off < k0;  // every query of the tile lies before this wavefront's keys
      if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) skip = skip || (qt0 + a.q_off - (k0 + 31) > a.window);
    }
    if (!skip) {
      const char* bias_base = a.aux.bias ? a.aux.bias + b * a.aux.bias_sb + h * a.aux.bias_sh : nullptr;
      const uint8_t* drop_base = a.aux.drop ? a.aux.drop + b * a.aux.drop_sb + h * a.aux.drop_sh : nullptr;
      floatx16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
      const float* q_row = q_lds + l32 * PS;
      const float* do_row = do_lds + l32 * PS;
#pragma unroll
      for (int d2 = 0; d2 < D / 2; d2++) {
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(q_row[2 * d2 + g], k_mine[d2], s, 0, 0, 0);
        dp = __builtin_amdgcn_mfma_f32_32x32x2f32(do_row[2 * d2 + g], v_row[2 * d2 + g], dp, 0, 0, 0);
      }
      floatx16 pd;  // probabilities after dropout, for dV
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int qi = 8 * (r / 4) + 4 * g + (r % 4);
        const int qpos = qt0 + qi + a.q_off;
        bool keep = true;
        if (a.mask_kind != AXL_MASK_NONE) {
          const int diff = qpos - kpos;
          keep = diff >= 0;
          if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) keep = keep && diff <= a.window;
        }
        if (seg_q) keep = keep && (seg_q[qt0 + qi] == seg_k);
        float logit = s[r] * a.scale;
        if (bias_base) logit += bias_at(a.aux, bias_base + (int64_t)(qt0 + qi) * a.aux.bias_sr, kpos);
        const float p = keep ? expf(logit - lse_lds[qi]) : 0.f;
        float dpe = dp[r];
        pd[r] = p;
        if (drop_base) {
          const bool dropped = drop_base[(int64_t)(qt0 + qi) * a.aux.drop_sr + kpos] != 0;
          dpe = dropped ? 0.f : dpe * a.aux.keep_scale;
          pd[r] = dropped ? 0.f : p * a.aux.keep_scale;
        }
        s[r] = p * (dpe - delta_lds[qi]);  // dS
      }
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int qi = 8 * (r / 4) + 4 * g + (r % 4);
        const float* do_col = do_lds + qi * PS + l32;
        const float* q_col = q_lds + qi * PS + l32;
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
          dv[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(do_col[32 * dt], pd[r], dv[dt], 0, 0, 0);
          dk[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(q_col[32 * dt], s[r], dk[dt], 0, 0, 0);
        }
      }
    }
    if (more) deposit(e + 1);  // the other buffer was last read a step ago, before the barrier that ended it
    __syncthreads();
  }

  float* dkp = (float*)a.dk + b * a.dks.b + (int64_t)kpos * a.dks.s + hk * a.dks.h;
  float* dvp = (float*)a.dv + b * a.dvs.b + (int64_t)kpos * a.dvs.s + hk * a.dvs.h;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int rq = 0; rq < 4; rq++) {
      float4 wk = {dk[dt][4 * rq + 0] * a.scale, dk[dt][4 * rq + 1] * a.scale, dk[dt][4 * rq + 2] * a.scale,
                   dk[dt][4 * rq + 3] * a.scale};
      float4 wv = {dv[dt][4 * rq + 0], dv[dt][4 * rq + 1], dv[dt][4 * rq + 2], dv[dt][4 * rq + 3]};
      *(float4*)(dkp + 32 * dt + 8 * rq + 4 * g) = wk;
      *(float4*)(dvp + 32 * dt + 8 * rq + 4 * g) = wv;
    }
}

// =============================================================================================
// The same two kernels with their fp32 products on the 16-bit matrix instruction (split3 / mfma_split in
// common.h: three bf16 parts per operand, six partial products per product, fp32 accumulation; this GPU
// multiplies bf16 sixteen times as fast as fp32).  Mapping and loop structure are those of the kernels
// above; operand layouts are those of the 16-bit kernels: a tile is kept in LDS as three 16-bit planes
// [row][d], read by rows (16 bytes at d = 16 s + 8 g of row swap_bits_2_3(l32): with that row order the
// registers 0..7 / 8..15 of an accumulator column are the rows 8g .. 8g+7 of the tile's first / second
// half, and, split and packed, are the B operand of the next product as they stand) and by transposing
// reads (row 8g + j16/4, +4, +16; columns 32 dt + 16 half + 4 (j16 % 4)).  Logits are kept in units of
// log2 (the stationary operand is multiplied by scale * log2(e) before its split, lse by log2(e)), the
// exponential is v_exp_f32.
// =============================================================================================
template <int D>
struct BwdTileF32x {
  static constexpr int NT = 256;
  static constexpr int ROWS = 128;
  static constexpr int TILE = 32;
  static constexpr int STRIDE = D * 2;                 // bytes per row of a tile plane: unpadded, 16-byte chunks swizzled
                                                       // (tile_swizzle: free of bank conflicts for both kinds of read)
  static constexpr int OWN_STRIDE = D * 2 + 16;        // rows of the owned planes, read one row per lane: padded
  static constexpr int PLANE = TILE * STRIDE;
  static constexpr int TENSOR = 3 * PLANE;
  static constexpr int BUF_BYTES = 2 * TENSOR + 2 * TILE * 4;   // two tensors' tiles, two rows of statistics
  static constexpr int PS = D + 1;                     // words per row of the fp32 pass of the owned rows
  static constexpr int OWN_BYTES = ROWS * PS * 4;
  static constexpr int LDS_BYTES = 2 * BUF_BYTES > OWN_BYTES ? 2 * BUF_BYTES : OWN_BYTES;
  static constexpr int OWN_PLANE = ROWS * OWN_STRIDE;   // one plane of an owned tensor kept in LDS (dK/dV kernel: K)
  static constexpr int LDS_BYTES_DKDV = 3 * OWN_PLANE + BUF_BYTES > OWN_BYTES ? 3 * OWN_PLANE + BUF_BYTES : OWN_BYTES;
  static constexpr int LD4 = TILE * (D / 4) / NT;
  static_assert(TILE * (D / 4) % NT == 0, "a tile divides evenly over the threads");
  static_assert(LDS_BYTES_DKDV <= 160 * 1024, "the owned K planes and one tile buffer fit the LDS");
};

// The workgroup's 128 owned rows of one tensor pass through LDS once as fp32; every lane keeps, multiplied
// by `mult` and split, elements 16 s + 8 g .. + 7 of its row.  Called by all threads; contains barriers.
template <int D>
__device__ __forceinline__ void own_rows_split(bf16x8 (&mine)[D / 16][3], float* lds, const float* src, int64_t stride,
                                               int tid, float mult) {
  using Tile = BwdTileF32x<D>;
  __syncthreads();  // whoever read this memory before is done
  for (int i = tid; i < Tile::ROWS * (D / 4); i += Tile::NT) {
    const int row = i / (D / 4), c4 = i % (D / 4);
    const float4 x = *(const float4*)(src + (int64_t)row * stride + c4 * 4);
    float* dst = lds + row * Tile::PS + c4 * 4;
    dst[0] = x.x; dst[1] = x.y; dst[2] = x.z; dst[3] = x.w;
  }
  __syncthreads();
  const int lane = tid & 63, g = lane >> 5;
  const float* row = lds + ((tid >> 6) * 32 + (lane & 31)) * Tile::PS;
#pragma unroll
  for (int s = 0; s < D / 16; s++) {
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; j++) x[j] = row[16 * s + 8 * g + j] * mult;
    Split3x8 sp;
    split3x8(x, sp);
#pragma unroll
    for (int p = 0; p < 3; p++) mine[s][p] = sp.part[p].v;
  }
}

// This thread's part of a 32 x D tile, split, into the tile's three planes.
template <int D>
__device__ __forceinline__ void tile_deposit_split(char* planes, const float4 (&x)[BwdTileF32x<D>::LD4], int tid) {
  using Tile = BwdTileF32x<D>;
#pragma unroll
  for (int i = 0; i < Tile::LD4; i++) {
    const int e = tid + i * Tile::NT, row = e / (D / 4), c4 = e % (D / 4);
    const Split3x2 lo2 = split3(x[i].x, x[i].y), hi2 = split3(x[i].z, x[i].w);
#pragma unroll
    for (int p = 0; p < 3; p++) {
      union { bf16x2 h[2]; uint2 u; } w;
      w.h[0] = lo2.part[p]; w.h[1] = hi2.part[p];
      *(uint2*)(planes + p * Tile::PLANE + row * Tile::STRIDE + (((c4 >> 1) ^ tile_swizzle<D>(row)) << 4) + (c4 & 1) * 8) = w.u;
    }
  }
}
template <int D>
__device__ __forceinline__ void tile_request_x(float4 (&x)[BwdTileF32x<D>::LD4], const float* src, int64_t stride, int tid) {
  using Tile = BwdTileF32x<D>;
#pragma unroll
  for (int i = 0; i < Tile::LD4; i++) {
    const int e = tid + i * Tile::NT, row = e / (D / 4), c4 = e % (D / 4);
    x[i] = *(const float4*)(src + (int64_t)row * stride + c4 * 4);
  }
}
// Per-lane read offsets into a tile plane.
template <int D>
struct TileReadOffsets {
  int row_base, row_xor;          // row read: row swap_bits_2_3(l32), chunk (2 ks + g) ^ swizzle
  int tr_base[2], tr_xor[2];      // transposing read: rows 8 g + j16 / 4 and + 4, byte column (16 half + 4 (j16 % 4)) * 2 + 64 dt
  int tr_col;
  __device__ __forceinline__ void init(int lane) {
    using Tile = BwdTileF32x<D>;
    const int l32 = lane & 31, g = lane >> 5, j16 = lane & 15, half = (lane >> 4) & 1;
    const int row = swap_bits_2_3(l32);
    row_base = row * Tile::STRIDE;
    row_xor = (16 * g) ^ (tile_swizzle<D>(row) << 4);
    const int t_row = 8 * g + (j16 >> 2), col = (16 * half + 4 * (j16 & 3)) * 2;
    tr_col = col & ~15;
    tr_base[0] = t_row * Tile::STRIDE + (col & 15);
    tr_base[1] = tr_base[0] + 4 * Tile::STRIDE;
    tr_xor[0] = tile_swizzle<D>(t_row) << 4;
    tr_xor[1] = tile_swizzle<D>(t_row + 4) << 4;
  }
};
// Row-read operand (A) of k-step `ks` from a tile's planes.
template <int D>
__device__ __forceinline__ void read_rows(bf16x8 (&f)[3], const char* planes, const TileReadOffsets<D>& o, int ks) {
#pragma unroll
  for (int p = 0; p < 3; p++) f[p] = *(const bf16x8*)(planes + p * BwdTileF32x<D>::PLANE + o.row_base + ((32 * ks) ^ o.row_xor));
}
// Transposed operand (A) for the tile's rows 16 kk + 8 g .. + 7 and columns 32 dt + l32.
template <int D>
__device__ __forceinline__ void read_transposed(bf16x8 (&f)[3], const char* planes, const TileReadOffsets<D>& o, int kk,
                                                int dt) {
  using Tile = BwdTileF32x<D>;
#pragma unroll
  for (int p = 0; p < 3; p++) {
    union { bf16x8 v; shortx4 hlf[2]; } u;
    const char* at = planes + p * Tile::PLANE + 16 * kk * Tile::STRIDE;   // rows + 16: the same swizzle
    u.hlf[0] = lds_read_tr16(at + o.tr_base[0] + ((o.tr_col + 64 * dt) ^ o.tr_xor[0]));
    u.hlf[1] = lds_read_tr16(at + o.tr_base[1] + ((o.tr_col + 64 * dt) ^ o.tr_xor[1]));
    f[p] = u.v;
  }
}
// Registers 8 kk .. 8 kk + 7 of an accumulator column, split: the B operand of the next product.
__device__ __forceinline__ void split_column(bf16x8 (&f)[3], const floatx16& acc, int kk) {
  float x[8];
#pragma unroll
  for (int j = 0; j < 8; j++) x[j] = acc[8 * kk + j];
  Split3x8 sp;
  split3x8(x, sp);
#pragma unroll
  for (int p = 0; p < 3; p++) f[p] = sp.part[p].v;
}

template <int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void flash_bwd_dq_f32x_kernel(const BwdArgs a) {
  using Tile = BwdTileF32x<D>;
  constexpr int DT = D / 32, KSTEPS = D / 16;
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  const int nqb = a.T / Tile::ROWS;
  const int qb = nqb - 1 - blockIdx.x % nqb;  // heaviest blocks of a causal mask first
  const int h = (blockIdx.x / nqb) % a.Hq, b = blockIdx.x / (nqb * a.Hq);
  const int hk = h / (a.Hq / a.Hkv);
  const int q0_wg = qb * Tile::ROWS, q0 = q0_wg + wave * 32;

  bf16x8 q_mine[KSTEPS][3], do_mine[KSTEPS][3];
  own_rows_split<D>(q_mine, (float*)smem, (const float*)a.q + b * a.qs.b + (int64_t)q0_wg * a.qs.s + h * a.qs.h, a.qs.s,
                    tid, a.scale * kLog2e);
  own_rows_split<D>(do_mine, (float*)smem, (const float*)a.dout + b * a.dos.b + (int64_t)q0_wg * a.dos.s + h * a.dos.h,
                    a.dos.s, tid, 1.f);
  const float* kp = (const float*)a.k + b * a.ks.b + hk * a.ks.h;
  const float* vp = (const float*)a.v + b * a.vs.b + hk * a.vs.h;
  const int64_t stat = ((int64_t)b * a.Hq + h) * a.T + q0 + l32;
  const float lse_q = a.lse[stat] * kLog2e, delta_q = -a.ndelta[stat];

  int k_begin = 0, k_end = a.S;
  if (a.mask_kind != AXL_MASK_NONE) {
    k_end = min(a.S, q0_wg + Tile::ROWS + a.q_off);
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) k_begin = max(0, q0_wg + a.q_off - a.window);
  }
  const int t_begin = k_begin / Tile::TILE;
  const int t_end = (k_end + Tile::TILE - 1) / Tile::TILE;
  const int qpos = q0 + l32 + a.q_off;
  const int qpos_min = q0 + a.q_off, qpos_max = q0 + 31 + a.q_off;
  const int seg_q = a.seg ? a.seg[(int64_t)b * a.T + q0 + l32] : 0;
  const int32_t* seg_k = a.seg ? a.seg + (int64_t)b * a.T : nullptr;
  const char* bias_row = nullptr;
  const uint8_t* drop_row = nullptr;
  if (a.aux.bias) bias_row = a.aux.bias + b * a.aux.bias_sb + h * a.aux.bias_sh + (int64_t)(q0 + l32) * a.aux.bias_sr;
  if (a.aux.drop) drop_row = a.aux.drop + b * a.aux.drop_sb + h * a.aux.drop_sh + (int64_t)(q0 + l32) * a.aux.drop_sr;

  floatx16 dq[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq[i][r] = 0.f;

  TileReadOffsets<D> off;
  off.init(lane);

  // Tile t lives in ring buffer t % 2: the planes of K, then of V.
  float4 kx[Tile::LD4], vx[Tile::LD4];
  __syncthreads();  // the owned rows have been read out of the memory
  if (t_begin < t_end) {
    tile_request_x<D>(kx, kp + (int64_t)t_begin * Tile::TILE * a.ks.s, a.ks.s, tid);
    tile_request_x<D>(vx, vp + (int64_t)t_begin * Tile::TILE * a.vs.s, a.vs.s, tid);
    char* buf = smem + (t_begin & 1) * Tile::BUF_BYTES;
    tile_deposit_split<D>(buf, kx, tid);
    tile_deposit_split<D>(buf + Tile::TENSOR, vx, tid);
  }
  __syncthreads();
  for (int t = t_begin; t < t_end; t++) {
    const int k0 = t * Tile::TILE;
    const bool more = t + 1 < t_end;
    if (more) {  // the next tile's round trip runs under this tile's MFMAs
      tile_request_x<D>(kx, kp + (int64_t)(k0 + Tile::TILE) * a.ks.s, a.ks.s, tid);
      tile_request_x<D>(vx, vp + (int64_t)(k0 + Tile::TILE) * a.vs.s, a.vs.s, tid);
    }
    const char* k_lds = smem + (t & 1) * Tile::BUF_BYTES;
    const char* v_lds = k_lds + Tile::TENSOR;
    bool skip = false;
    if (a.mask_kind != AXL_MASK_NONE) {
      skip = k0 > qpos_max;
      if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) skip = skip || (qpos_min - (k0 + Tile::TILE - 1) > a.window);
    }
    if (!skip) {
      floatx16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) {
        bf16x8 kf[3], vf[3];
        read_rows<D>(kf, k_lds, off, ks);
        read_rows<D>(vf, v_lds, off, ks);
        s = mfma_split(kf, q_mine[ks], s);
        dp = mfma_split(vf, do_mine[ks], dp);
      }
      // Register r of lane group g is key k0 + 16 (r / 8) + 8 g + r % 8.  A tile in the interior of the
      // wavefront's range (every key at or before its first query and inside the window of its last one),
      // without segment ids, bias or dropout mask, has nothing to mask or to look up.
      bool interior = seg_k == nullptr && bias_row == nullptr && drop_row == nullptr;
      if (a.mask_kind != AXL_MASK_NONE) {
        interior = interior && k0 + Tile::TILE - 1 <= qpos_min;
        if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) interior = interior && qpos_max - k0 <= a.window;
      }
      if (interior) {
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = fast_exp2(s[r] - lse_q) * (dp[r] - delta_q);  // dS^T
      } else {
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
          float logit = s[r];
          if (bias_row) logit += bias_at(a.aux, bias_row, kpos) * kLog2e;
          const float p = keep ? fast_exp2(logit - lse_q) : 0.f;
          float dpe = dp[r];
          if (drop_row) dpe = drop_row[kpos] ? 0.f : dpe * a.aux.keep_scale;
          s[r] = p * (dpe - delta_q);  // dS^T
        }
      }
      // dQ^T[d][q] += K^T[d][key] dS^T[key][q], 16 keys per step.
#pragma unroll
      for (int kk = 0; kk < 2; kk++) {
        bf16x8 dsf[3];
        split_column(dsf, s, kk);
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
          bf16x8 kt[3];
          read_transposed<D>(kt, k_lds, off, kk, dt);
          dq[dt] = mfma_split(kt, dsf, dq[dt]);
        }
      }
    }
    if (more) {  // the other buffer was last read a tile ago, before the barrier that ended that tile
      char* buf = smem + ((t + 1) & 1) * Tile::BUF_BYTES;
      tile_deposit_split<D>(buf, kx, tid);
      tile_deposit_split<D>(buf + Tile::TENSOR, vx, tid);
    }
    __syncthreads();
  }

  float* dqp = (float*)a.dq + b * a.dqs.b + (int64_t)(q0 + l32) * a.dqs.s + h * a.dqs.h;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int rq = 0; rq < 4; rq++) {
      float4 w = {dq[dt][4 * rq + 0] * a.scale, dq[dt][4 * rq + 1] * a.scale, dq[dt][4 * rq + 2] * a.scale,
                  dq[dt][4 * rq + 3] * a.scale};
      *(float4*)(dqp + 32 * dt + 8 * rq + 4 * g) = w;
    }
}

template <int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void flash_bwd_dkdv_f32x_kernel(const BwdArgs a) {
  using Tile = BwdTileF32x<D>;
  constexpr int DT = D / 32, KSTEPS = D / 16;
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  const int nkb = a.S / Tile::ROWS;
  const int kb = blockIdx.x % nkb;
  const int hk = (blockIdx.x / nkb) % a.Hkv, b = blockIdx.x / (nkb * a.Hkv);
  const int G = a.Hq / a.Hkv;
  const int k0_wg = kb * Tile::ROWS, k0 = k0_wg + wave * 32;
  const int kpos = k0 + l32;

  // The owned V rows live, split, in registers; the owned K rows (times scale * log2(e)), split, in three
  // planes in LDS behind which a single tile buffer follows: both in registers would not fit beside the
  // two accumulator sets, and two tile buffers would not fit beside the planes.
  bf16x8 v_mine[KSTEPS][3];
  own_rows_split<D>(v_mine, (float*)smem, (const float*)a.v + b * a.vs.b + (int64_t)k0_wg * a.vs.s + hk * a.vs.h, a.vs.s,
                    tid, 1.f);
  __syncthreads();  // the fp32 pass has been read
  {
    const float* src = (const float*)a.k + b * a.ks.b + (int64_t)k0_wg * a.ks.s + hk * a.ks.h;
    const float c = a.scale * kLog2e;
    for (int i = tid; i < Tile::ROWS * (D / 4); i += Tile::NT) {
      const int row = i / (D / 4), c4 = i % (D / 4);
      const float4 x = *(const float4*)(src + (int64_t)row * a.ks.s + c4 * 4);
      const Split3x2 lo2 = split3(x.x * c, x.y * c), hi2 = split3(x.z * c, x.w * c);
#pragma unroll
      for (int p = 0; p < 3; p++) {
        union { bf16x2 h[2]; uint2 u; } w;
        w.h[0] = lo2.part[p]; w.h[1] = hi2.part[p];
        *(uint2*)(smem + p * Tile::OWN_PLANE + row * Tile::OWN_STRIDE + c4 * 8) = w.u;
      }
    }
  }
  const char* const k_own = smem + (wave * 32 + l32) * Tile::OWN_STRIDE + 16 * g;   // this lane's key, d = 8 g ..
  char* const tile_buf = smem + 3 * Tile::OWN_PLANE;

  // Query rows that can see a key of this block: qpos >= first key, qpos <= last key + window.
  int q_begin = 0, q_end = a.T;
  if (a.mask_kind != AXL_MASK_NONE) {
    q_begin = min(a.T, max(0, k0_wg - a.q_off));
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW)
      q_end = max(q_begin, (int)min((int64_t)a.T, (int64_t)k0_wg + Tile::ROWS + a.window - a.q_off));
  }
  const int t_begin = q_begin / Tile::TILE;
  const int t_end = (q_end + Tile::TILE - 1) / Tile::TILE;
  const int nt = max(t_end - t_begin, 0);
  const int seg_k = a.seg ? a.seg[(int64_t)b * a.T + kpos] : 0;
  const int32_t* seg_q = a.seg ? a.seg + (int64_t)b * a.T : nullptr;

  floatx16 dk[DT], dv[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dk[i][r] = dv[i][r] = 0.f;

  TileReadOffsets<D> off;
  off.init(lane);

  // Step e of the loop is query tile t_begin + e % nt of query head hk G + e / nt: the planes of Q, then
  // of dO, then lse (in log2 units) and delta of the 32 queries.
  const int steps = nt * G;
  float4 qx[Tile::LD4], dox[Tile::LD4];
  float stat_x = 0.f;  // threads 0..31: lse, 32..63: delta of query tid % 32
  auto request = [&](int e) __attribute__((always_inline)) {
    const int h = hk * G + e / nt, qt0 = (t_begin + e % nt) * Tile::TILE;
    tile_request_x<D>(qx, (const float*)a.q + b * a.qs.b + h * a.qs.h + (int64_t)qt0 * a.qs.s, a.qs.s, tid);
    tile_request_x<D>(dox, (const float*)a.dout + b * a.dos.b + h * a.dos.h + (int64_t)qt0 * a.dos.s, a.dos.s, tid);
    const int64_t row = ((int64_t)b * a.Hq + h) * a.T + qt0 + (tid & 31);
    if (tid < 32) stat_x = a.lse[row] * kLog2e;
    else if (tid < 64) stat_x = -a.ndelta[row];
  };
  auto deposit = [&]() __attribute__((always_inline)) {
    char* buf = tile_buf;
    tile_deposit_split<D>(buf, qx, tid);
    tile_deposit_split<D>(buf + Tile::TENSOR, dox, tid);
    if (tid < 64) ((float*)(buf + 2 * Tile::TENSOR))[tid] = stat_x;
  };
  if (steps > 0) {
    request(0);
    deposit();
  }
  __syncthreads();  // the K planes and the first tile are in place
  for (int e = 0; e < steps; e++) {
    const int h = hk * G + e / nt, qt0 = (t_begin + e % nt) * Tile::TILE;
    const bool more = e + 1 < steps;
    if (more) request(e + 1);  // the next tile's round trip runs under this tile's MFMAs
    const char* q_lds = tile_buf;
    const char* do_lds = q_lds + Tile::TENSOR;
    const float* lse_lds = (const float*)(q_lds + 2 * Tile::TENSOR);
    const float* delta_lds = lse_lds + Tile::TILE;
    bool skip = false;
    if (a.mask_kind != AXL_MASK_NONE) {
      skip = qt0 + 31 + a.q_off < k0;  // every query of the tile lies before this wavefront's keys
      if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) skip = skip || (qt0 + a.q_off - (k0 + 31) > a.window);
    }
    if (!skip) {
      const char* bias_base = a.aux.bias ? a.aux.bias + b * a.aux.bias_sb + h * a.aux.bias_sh : nullptr;
      const uint8_t* drop_base = a.aux.drop ? a.aux.drop + b * a.aux.drop_sb + h * a.aux.drop_sh : nullptr;
      // S[q][key] = Q K^T, dP[q][key] = dO V^T: A = rows of the tile, B = this lane's key.
      floatx16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) {
        bf16x8 qf[3], dof[3];
        read_rows<D>(qf, q_lds, off, ks);
        read_rows<D>(dof, do_lds, off, ks);
        bf16x8 kf[3];
#pragma unroll
        for (int p = 0; p < 3; p++) kf[p] = *(const bf16x8*)(k_own + p * Tile::OWN_PLANE + 32 * ks);
        s = mfma_split(qf, kf, s);
        dp = mfma_split(dof, v_mine[ks], dp);
      }
      // Register r of lane group g is query qt0 + 16 (r / 8) + 8 g + r % 8.  Afterwards s holds dS and dp
      // the probabilities (after dropout) that dV takes.  A tile all of whose queries see all of the
      // wavefront's keys, without segment ids, bias or dropout mask, has nothing to mask or to look up.
      bool interior = seg_q == nullptr && bias_base == nullptr && drop_base == nullptr;
      if (a.mask_kind != AXL_MASK_NONE) {
        interior = interior && qt0 + a.q_off >= k0 + 31;
        if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) interior = interior && qt0 + 31 + a.q_off - k0 <= a.window;
      }
      if (interior) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int qi = 16 * (r / 8) + 8 * g + (r % 8);
          const float p = fast_exp2(s[r] - lse_lds[qi]);
          s[r] = p * (dp[r] - delta_lds[qi]);  // dS
          dp[r] = p;
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int qi = 16 * (r / 8) + 8 * g + (r % 8);
          const int qpos = qt0 + qi + a.q_off;
          bool keep = true;
          if (a.mask_kind != AXL_MASK_NONE) {
            const int diff = qpos - kpos;
            keep = diff >= 0;
            if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) keep = keep && diff <= a.window;
          }
          if (seg_q) keep = keep && (seg_q[qt0 + qi] == seg_k);
          float logit = s[r];
          if (bias_base) logit += bias_at(a.aux, bias_base + (int64_t)(qt0 + qi) * a.aux.bias_sr, kpos) * kLog2e;
          const float p = keep ? fast_exp2(logit - lse_lds[qi]) : 0.f;
          float dpe = dp[r], pd = p;
          if (drop_base) {
            const bool dropped = drop_base[(int64_t)(qt0 + qi) * a.aux.drop_sr + kpos] != 0;
            dpe = dropped ? 0.f : dpe * a.aux.keep_scale;
            pd = dropped ? 0.f : p * a.aux.keep_scale;
          }
          s[r] = p * (dpe - delta_lds[qi]);  // dS
          dp[r] = pd;
        }
      }
      // dV^T[d][key] += dO^T[d][q] P[q][key],  dK^T[d][key] += Q^T[d][q] dS[q][key], 16 queries per step.
#pragma unroll
      for (int kk = 0; kk < 2; kk++) {
        bf16x8 pf[3], dsf[3];
        split_column(pf, dp, kk);
        split_column(dsf, s, kk);
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
          bf16x8 dot[3], qt[3];
          read_transposed<D>(dot, do_lds, off, kk, dt);
          read_transposed<D>(qt, q_lds, off, kk, dt);
          dv[dt] = mfma_split(dot, pf, dv[dt]);
          dk[dt] = mfma_split(qt, dsf, dk[dt]);
        }
      }
    }
    __syncthreads();  // every wavefront has read the tile
    if (more) deposit();
    __syncthreads();
  }

  float* dkp = (float*)a.dk + b * a.dks.b + (int64_t)kpos * a.dks.s + hk * a.dks.h;
  float* dvp = (float*)a.dv + b * a.dvs.b + (int64_t)kpos * a.dvs.s + hk * a.dvs.h;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int rq = 0; rq < 4; rq++) {
      float4 wk = {dk[dt][4 * rq + 0] * a.scale, dk[dt][4 * rq + 1] * a.scale, dk[dt][4 * rq + 2] * a.scale,
                   dk[dt][4 * rq + 3] * a.scale};
      float4 wv = {dv[dt][4 * rq + 0], dv[dt][4 * rq + 1], dv[dt][4 * rq + 2], dv[dt][4 * rq + 3]};
      *(float4*)(dkp + 32 * dt + 8 * rq + 4 * g) = wk;
      *(float4*)(dvp + 32 * dt + 8 * rq + 4 * g) = wv;
    }
}

template <int D>
static hipError_t launch_f32(const BwdArgs& a, int phases, hipStream_t stream) {
  using Tile = BwdTileF32<D>;
  using TileX = BwdTileF32x<D>;
  // AXL_F32_MFMA=1 in the environment: the kernels on the fp32 matrix instruction (for comparison).
  static const bool true_f32 = [] { const char* e = getenv("AXL_F32_MFMA"); return e && e[0] == '1'; }();
  hipError_t err = hipSuccess;
  if (phases & AXL_BWD_DKDV) {
    auto kernel = true_f32 ? flash_bwd_dkdv_f32_kernel<D> : flash_bwd_dkdv_f32x_kernel<D>;
    const int lds = true_f32 ? Tile::LDS_BYTES_DKDV : TileX::LDS_BYTES_DKDV;
    err = allow_dynamic_lds((const void*)kernel, lds);
    if (err != hipSuccess) return err;
    hipLaunchKernelGGL(kernel, dim3((a.S / Tile::ROWS) * a.B * a.Hkv), dim3(Tile::NT), lds, stream, a);
    err = hipGetLastError();
    if (err != hipSuccess) return err;
  }
  if (phases & AXL_BWD_DQ) {
    auto kernel = true_f32 ? flash_bwd_dq_f32_kernel<D> : flash_bwd_dq_f32x_kernel<D>;
    const int lds = true_f32 ? Tile::LDS_BYTES : TileX::LDS_BYTES;
    err = allow_dynamic_lds((const void*)kernel, lds);
    if (err != hipSuccess) return err;
    hipLaunchKernelGGL(kernel, dim3((a.T / Tile::ROWS) * a.B * a.Hq), dim3(Tile::NT), lds, stream, a);
    err = hipGetLastError();
  }
  return err;
}

hipError_t launch_bwd_f32(const BwdArgs& a, int head_dim, int phases, hipStream_t stream) {
  return head_dim == 128 ? launch_f32<128>(a, phases, stream) : launch_f32<64>(a, phases, stream);
}

}  // namespace axl
