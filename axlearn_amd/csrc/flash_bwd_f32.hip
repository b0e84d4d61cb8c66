// fp32 flash-attention backward for gfx950: dQ and dK/dV with v_mfma_f32_32x32x2_f32 (true fp32
// multiply-accumulate) and the accurate exponential.
//
// Replaces the float32 case of axlearn/common/flash_attention/gpu_attention.py:621-786
// (`_mha_backward`, which shrinks its blocks to 32 for float32 inputs, :645-646, and whose tests run
// float32 forward + backward, gpu_attention_test.py:197) with
//   p  = exp(scale * q k^T + bias - lse)                    (:507, :599)
//   dp = dO v^T, zeroed where dropped and scaled by 1/(1-rate)   (:508-512, :600-603)
//   ds = p * (dp - delta)                                   (:514, :604)
//   dv += (p after dropout)^T dO,  dk += scale * ds^T q,  dq += scale * ds k   (:513, :518, :608)
// This path is for parity, not speed: tiles are staged through LDS by ordinary loads, one 32-row
// tile per step, nothing is pipelined.  The mapping is the forward's (flash_fwd.hip, fp32 kernel):
// an accumulator register r of lane (l32, g) is row 8(r/4) + 4g + (r%4), column l32, so a product
// whose reduction runs over the accumulator's rows takes register r itself as the B operand of
// MFMA r ("one reduction index per lane group per MFMA").
#include "flash_bwd.h"

namespace axl {

template <int D>
struct BwdTileF32 {
  static constexpr int ROWS = 64;              // rows owned by a workgroup (2 wavefronts x 32)
  static constexpr int TILE = 32;              // rows of the tiles it loops over
  static constexpr int PS = D + 1;             // words per LDS row: lanes read a column of rows
  static constexpr int LDS_BYTES = (2 * ROWS + 2 * TILE) * PS * 4 + 2 * TILE * 4;
};

// rows x D floats from global (row stride `stride` elements) into LDS rows of PS words.
template <int D, int NT>
__device__ __forceinline__ void stage_rows(float* lds, const float* src, int64_t stride, int rows, int tid) {
  constexpr int PS = D + 1;
  for (int i = tid; i < rows * (D / 4); i += NT) {
    const int row = i / (D / 4), c4 = i % (D / 4);
    const float4 x = *(const float4*)(src + (int64_t)row * stride + c4 * 4);
    float* dst = lds + row * PS + c4 * 4;
    dst[0] = x.x; dst[1] = x.y; dst[2] = x.z; dst[3] = x.w;
  }
}

__device__ __forceinline__ float bias_at(const AuxArgs& x, const char* row, int col) {
  if (x.bias_f32) return *(const float*)(row + (int64_t)col * 4);
  return (float)*(const __bf16*)(row + (int64_t)col * 2);
}

// ---------------------------------------------------------------------------------------------
// dQ: a workgroup owns 64 query rows of one head and loops over 32-key tiles.
//   S^T[key][q] = K Q^T and dP^T[key][q] = V dO^T (A = K / V row l32, B = Q / dO row l32), so lane
//   (l32, g) holds query l32 and keys 8(r/4) + 4g + (r%4); dQ^T[d][q] += K^T[d][key] dS^T[key][q].
// ---------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(128) void flash_bwd_dq_f32_kernel(const BwdArgs a) {
  using Tile = BwdTileF32<D>;
  constexpr int DT = D / 32, PS = Tile::PS;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* const q_lds = (float*)smem;
  float* const do_lds = q_lds + Tile::ROWS * PS;
  float* const k_lds = do_lds + Tile::ROWS * PS;
  float* const v_lds = k_lds + Tile::TILE * PS;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  const int nqb = a.T / Tile::ROWS;
  const int qb = nqb - 1 - blockIdx.x % nqb;  // heaviest blocks of a causal mask first
  const int h = (blockIdx.x / nqb) % a.Hq, b = blockIdx.x / (nqb * a.Hq);
  const int hk = h / (a.Hq / a.Hkv);
  const int q0_wg = qb * Tile::ROWS, q0 = q0_wg + wave * 32;

  stage_rows<D, 128>(q_lds, (const float*)a.q + b * a.qs.b + (int64_t)q0_wg * a.qs.s + h * a.qs.h, a.qs.s,
                     Tile::ROWS, tid);
  stage_rows<D, 128>(do_lds, (const float*)a.dout + b * a.dos.b + (int64_t)q0_wg * a.dos.s + h * a.dos.h, a.dos.s,
                     Tile::ROWS, tid);
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
  const float* q_row = q_lds + (wave * 32 + l32) * PS;
  const float* do_row = do_lds + (wave * 32 + l32) * PS;

  for (int t = t_begin; t < t_end; t++) {
    const int k0 = t * Tile::TILE;
    __syncthreads();  // previous tile consumed (and Q, dO staged on the first pass)
    stage_rows<D, 128>(k_lds, kp + (int64_t)k0 * a.ks.s, a.ks.s, Tile::TILE, tid);
    stage_rows<D, 128>(v_lds, vp + (int64_t)k0 * a.vs.s, a.vs.s, Tile::TILE, tid);
    __syncthreads();
    bool skip = false;
    if (a.mask_kind != AXL_MASK_NONE) {
      skip = k0 > qpos_max;
      if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) skip = skip || (qpos_min - (k0 + Tile::TILE - 1) > a.window);
    }
    if (skip) continue;
    floatx16 s, dp;
#pragma unroll
    for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
    const float* k_row = k_lds + l32 * PS;
    const float* v_row = v_lds + l32 * PS;
#pragma unroll 8
    for (int d2 = 0; d2 < D / 2; d2++) {
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(k_row[2 * d2 + g], q_row[2 * d2 + g], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x2f32(v_row[2 * d2 + g], do_row[2 * d2 + g], dp, 0, 0, 0);
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
// dK/dV: a workgroup owns 64 keys of one kv head and loops over the query heads of its group and
// over 32-query tiles.
//   S[q][key] = Q K^T and dP[q][key] = dO V^T (A = Q / dO row l32 of the tile, B = K / V row l32), so
//   lane (l32, g) holds key l32 and queries 8(r/4) + 4g + (r%4);
//   dV^T[d][key] += dO^T[d][q] P[q][key],  dK^T[d][key] += Q^T[d][q] dS[q][key].
// ---------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(128) void flash_bwd_dkdv_f32_kernel(const BwdArgs a) {
  using Tile = BwdTileF32<D>;
  constexpr int DT = D / 32, PS = Tile::PS;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* const k_lds = (float*)smem;
  float* const v_lds = k_lds + Tile::ROWS * PS;
  float* const q_lds = v_lds + Tile::ROWS * PS;
  float* const do_lds = q_lds + Tile::TILE * PS;
  float* const lse_lds = do_lds + Tile::TILE * PS;
  float* const delta_lds = lse_lds + Tile::TILE;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  const int nkb = a.S / Tile::ROWS;
  const int kb = blockIdx.x % nkb;
  const int hk = (blockIdx.x / nkb) % a.Hkv, b = blockIdx.x / (nkb * a.Hkv);
  const int G = a.Hq / a.Hkv;
  const int k0_wg = kb * Tile::ROWS, k0 = k0_wg + wave * 32;
  const int kpos = k0 + l32;

  stage_rows<D, 128>(k_lds, (const float*)a.k + b * a.ks.b + (int64_t)k0_wg * a.ks.s + hk * a.ks.h, a.ks.s,
                     Tile::ROWS, tid);
  stage_rows<D, 128>(v_lds, (const float*)a.v + b * a.vs.b + (int64_t)k0_wg * a.vs.s + hk * a.vs.h, a.vs.s,
                     Tile::ROWS, tid);

  // Query rows that can see a key of this block: qpos >= first key, qpos <= last key + window.
  int q_begin = 0, q_end = a.T;
  if (a.mask_kind != AXL_MASK_NONE) {
    q_begin = min(a.T, max(0, k0_wg - a.q_off));
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW)
      q_end = max(q_begin, (int)min((int64_t)a.T, (int64_t)k0_wg + Tile::ROWS + a.window - a.q_off));
  }
  const int t_begin = q_begin / Tile::TILE;
  const int t_end = (q_end + Tile::TILE - 1) / Tile::TILE;
  const int seg_k = a.seg ? a.seg[(int64_t)b * a.T + kpos] : 0;
  const int32_t* seg_q = a.seg ? a.seg + (int64_t)b * a.T : nullptr;

  floatx16 dk[DT], dv[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dk[i][r] = dv[i][r] = 0.f;
  const float* k_row = k_lds + (wave * 32 + l32) * PS;
  const float* v_row = v_lds + (wave * 32 + l32) * PS;

  for (int hh = 0; hh < G; hh++) {
    const int h = hk * G + hh;
    const float* qp = (const float*)a.q + b * a.qs.b + h * a.qs.h;
    const float* dop = (const float*)a.dout + b * a.dos.b + h * a.dos.h;
    const int64_t stat = ((int64_t)b * a.Hq + h) * a.T;
    const char* bias_base = a.aux.bias ? a.aux.bias + b * a.aux.bias_sb + h * a.aux.bias_sh : nullptr;
    const uint8_t* drop_base = a.aux.drop ? a.aux.drop + b * a.aux.drop_sb + h * a.aux.drop_sh : nullptr;
    for (int t = t_begin; t < t_end; t++) {
      const int qt0 = t * Tile::TILE;
      __syncthreads();  // previous tile consumed (and K, V staged on the first pass)
      stage_rows<D, 128>(q_lds, qp + (int64_t)qt0 * a.qs.s, a.qs.s, Tile::TILE, tid);
      stage_rows<D, 128>(do_lds, dop + (int64_t)qt0 * a.dos.s, a.dos.s, Tile::TILE, tid);
      if (tid < Tile::TILE) {
        lse_lds[tid] = a.lse[stat + qt0 + tid];
        delta_lds[tid] = -a.ndelta[stat + qt0 + tid];
      }
      __syncthreads();
      bool skip = false;
      if (a.mask_kind != AXL_MASK_NONE) {
        skip = qt0 + 31 + a.q_off < k0;  // every query of the tile lies before this wavefront's keys
        if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) skip = skip || (qt0 + a.q_off - (k0 + 31) > a.window);
      }
      if (skip) continue;
      floatx16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
      const float* q_row = q_lds + l32 * PS;
      const float* do_row = do_lds + l32 * PS;
#pragma unroll 8
      for (int d2 = 0; d2 < D / 2; d2++) {
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(q_row[2 * d2 + g], k_row[2 * d2 + g], s, 0, 0, 0);
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
  hipError_t err = hipSuccess;
  if (phases & AXL_BWD_DKDV) {
    auto kernel = flash_bwd_dkdv_f32_kernel<D>;
    err = allow_dynamic_lds((const void*)kernel, Tile::LDS_BYTES);
    if (err != hipSuccess) return err;
    hipLaunchKernelGGL(kernel, dim3((a.S / Tile::ROWS) * a.B * a.Hkv), dim3(128), Tile::LDS_BYTES, stream, a);
    err = hipGetLastError();
    if (err != hipSuccess) return err;
  }
  if (phases & AXL_BWD_DQ) {
    auto kernel = flash_bwd_dq_f32_kernel<D>;
    err = allow_dynamic_lds((const void*)kernel, Tile::LDS_BYTES);
    if (err != hipSuccess) return err;
    hipLaunchKernelGGL(kernel, dim3((a.T / Tile::ROWS) * a.B * a.Hq), dim3(128), Tile::LDS_BYTES, stream, a);
    err = hipGetLastError();
  }
  return err;
}

hipError_t launch_bwd_f32(const BwdArgs& a, int head_dim, int phases, hipStream_t stream) {
  return head_dim == 128 ? launch_f32<128>(a, phases, stream) : launch_f32<64>(a, phases, stream);
}

}  // namespace axl
