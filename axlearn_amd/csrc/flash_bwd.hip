// Flash-attention backward for gfx950: delta pre-pass, dK/dV kernel, dQ kernel.
//
// Replaces axlearn/common/flash_attention/gpu_attention.py:621-786 (`_mha_backward`):
//   delta = rowsum(out * dO) in fp32                                   (:653-658)
//   `_mha_backward_kernel_dkdv` (:436-528):  p = exp(qk - lse); dv += p^T dO;
//        dp = dO v^T; ds = p * (dp - delta) * scale; dk += ds^T q
//   `_mha_backward_kernel_dq`  (:533-616):  dq += ds k
// p and ds are rounded to bf16 before their MFMAs, accumulation is fp32, as in the reference
// (:513, :518, :608).
//
// Machine mapping (all GEMMs are v_mfma_f32_32x32x16_bf16):
//   dK/dV: a workgroup owns 128 keys of one (batch, kv head); each wavefront keeps the K and V
//     fragments of its 32 keys in registers as B operands, streams 32-query Q/dO tiles through LDS,
//     and loops over ALL query heads of the kv head's group, so dK/dV need no atomics and no
//     repeated-KV reduction pass.  S = Q K^T and dP = dO V^T land with lane = key and
//     registers = queries; exp(S) and dS are then already B operands for dV^T += dO^T P and
//     dK^T += Q^T dS, whose A operands are transposing LDS reads of the same dO / Q tiles.
//   dQ: a workgroup owns 128 queries (32 per wavefront, Q and dO fragments in registers) and
//     streams 64-key K/V tiles through LDS exactly like the forward; S^T = K Q^T, dP^T = V dO^T,
//     dQ^T += K^T dS^T with K^T from transposing LDS reads.
#include "flash_bwd.h"

namespace axl {

// ---------------------------------------------------------------------------------------------
// delta[b,h,t] = sum_d out[b,t,h,d] * dO[b,t,h,d]; 16 lanes per row, 16 bytes per lane per step.
// Also leaves lse2 = -lse * log2(e) next to it: the dK/dV kernel streams both rows of statistics
// into LDS with direct loads, which cannot scale on the way.
// ---------------------------------------------------------------------------------------------
template <typename T, int D>
__global__ __launch_bounds__(256) void bwd_delta_kernel(const BwdArgs a) {
  constexpr int VEC = 16 / sizeof(T);         // elements per 16-byte load
  constexpr int STEPS = D / (16 * VEC);       // loads per lane to cover a row with 16 lanes
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);  // over B*T*Hq
  const int sub = threadIdx.x & 15;
  const int64_t rows = (int64_t)a.B * a.T * a.Hq;
  float acc = 0.f;
  int b = 0, t = 0, h = 0;
  if (row < rows) {
    h = (int)(row % a.Hq);
    t = (int)((row / a.Hq) % a.T);
    b = (int)(row / ((int64_t)a.Hq * a.T));
    const T* o = (const T*)a.out + b * a.os.b + (int64_t)t * a.os.s + h * a.os.h;
    const T* d = (const T*)a.dout + b * a.dos.b + (int64_t)t * a.dos.s + h * a.dos.h;
#pragma unroll
    for (int s = 0; s < (STEPS > 0 ? STEPS : 1); s++) {
      const int off = (s * 16 + sub) * VEC;
      if (off < a.d_real) {
        union { uint4 u; T e[VEC]; } x, y;
        x.u = *(const uint4*)(o + off);
        y.u = *(const uint4*)(d + off);
#pragma unroll
        for (int i = 0; i < VEC; i++) acc += (float)x.e[i] * (float)y.e[i];
      }
    }
  }
  acc += __shfl_xor(acc, 1, 64);
  acc += __shfl_xor(acc, 2, 64);
  acc += __shfl_xor(acc, 4, 64);
  acc += __shfl_xor(acc, 8, 64);
  if (row < rows && sub == 0) {
    const int64_t idx = ((int64_t)b * a.Hq + h) * a.T + t;
    a.ndelta[idx] = -acc;
    a.lse2[idx] = lse_to_exp2_offset(a.lse[idx]);
  }
}

// ---------------------------------------------------------------------------------------------
// Gradient of the per-head sink logit.  The sink's probability in row (b, h, t) is
// exp(sink[h] - lse[b,h,t]) and it has no value row (dP = 0), so dL/dsink is
// -sum_{b,t} exp(sink[h] - lse) * delta.  One workgroup per head; fixed summation order.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void bwd_dsink_kernel(const float* __restrict__ sink,
                                                        const float* __restrict__ lse,
                                                        const float* __restrict__ ndelta,
                                                        float* __restrict__ d_sink, int B, int Hq,
                                                        int T) {
  __shared__ float red[256];
  const int h = blockIdx.x, tid = threadIdx.x;
  const float sk = sink[h];
  float acc = 0.f;
  for (int b = 0; b < B; b++) {
    const int64_t base = ((int64_t)b * Hq + h) * T;
    for (int t = tid; t < T; t += 256) acc += expf(sk - lse[base + t]) * ndelta[base + t];
  }
  red[tid] = acc;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (tid < w) red[tid] += red[tid + w];
    __syncthreads();
  }
  if (tid == 0) d_sink[h] = red[0];
}

// ---------------------------------------------------------------------------------------------
// dQ.
// ---------------------------------------------------------------------------------------------
template <int D>
struct DqTile {
  static constexpr int BQ = 128;
  static constexpr int BK = 64;
  static constexpr int STRIDE = D * 2 + 16;
  static constexpr int TILE_BYTES = BK * STRIDE;
  static constexpr int CHUNKS = BK * D * 2 / 16 / 256;
  static constexpr int LDS_BYTES = 4 * TILE_BYTES;  // {K, V} x double buffer
};

template <typename E, int D, bool AUX>
__global__ __launch_bounds__(256) void flash_bwd_dq_aux_kernel(const BwdArgs a) {
  using Tile = DqTile<D>;
  constexpr int KK = D / 16, DT = D / 32;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* const k_lds = smem;
  char* const v_lds = smem + 2 * Tile::TILE_BYTES;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  const int nqb = a.T / Tile::BQ;
  const int per_qb = a.B * a.Hq;
  const int qb = nqb - 1 - blockIdx.x / per_qb;
  const int rem = blockIdx.x % per_qb;
  const int b = rem / a.Hq, h = rem % a.Hq;
  const int hk = h / (a.Hq / a.Hkv);
  const int q0_wg = qb * Tile::BQ;
  const int q0 = q0_wg + wave * 32;

  const __bf16* qp = (const __bf16*)a.q + b * a.qs.b + (int64_t)(q0 + l32) * a.qs.s + h * a.qs.h;
  const __bf16* dop = (const __bf16*)a.dout + b * a.dos.b + (int64_t)(q0 + l32) * a.dos.s + h * a.dos.h;
  const __bf16* kp = (const __bf16*)a.k + b * a.ks.b + hk * a.ks.h;
  const __bf16* vp = (const __bf16*)a.v + b * a.vs.b + hk * a.vs.h;
  bf16x8 qf[KK], dof[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) {
    qf[kk] = *(const bf16x8*)(qp + 16 * kk + 8 * g);
    dof[kk] = *(const bf16x8*)(dop + 16 * kk + 8 * g);
  }
  const int64_t stat_idx = ((int64_t)b * a.Hq + h) * a.T + q0 + l32;
  const float lse2 = -lse_to_exp2_offset(a.lse[stat_idx]);
  const float delta = -a.ndelta[stat_idx];

  int k_begin = 0, k_end = a.S;
  if (a.mask_kind != AXL_MASK_NONE) {
    k_end = min(a.S, q0_wg + Tile::BQ + a.q_off);
    if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) k_begin = max(0, q0_wg + a.q_off - a.window);
  }
  const int seg_q = a.seg ? a.seg[(int64_t)b * a.T + q0 + l32] : 0;
  const int32_t* seg_k = a.seg ? a.seg + (int64_t)b * a.T : nullptr;
  if (seg_k) shrink_to_segment_hull(seg_q, seg_k, tid, k_begin, k_end);
  const int t_begin = k_begin / Tile::BK;
  const int t_end = (k_end + Tile::BK - 1) / Tile::BK;
  const int qpos = q0 + l32 + a.q_off;
  const int qpos_min = q0 + a.q_off, qpos_max = q0 + 31 + a.q_off;
  const char* bias_row = nullptr;   // dense bias / dropout mask rows of this lane's query
  const uint8_t* drop_row = nullptr;
  if constexpr (AUX) {
    if (a.aux.bias) bias_row = a.aux.bias + b * a.aux.bias_sb + h * a.aux.bias_sh + (int64_t)(q0 + l32) * a.aux.bias_sr;
    if (a.aux.drop) drop_row = a.aux.drop + b * a.aux.drop_sb + h * a.aux.drop_sh + (int64_t)(q0 + l32) * a.aux.drop_sr;
  }

  floatx16 dq_acc[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq_acc[i][r] = 0.f;
  const float c = a.scale * kLog2e;

  // Global -> LDS staging through registers (plain unrolled code so the arrays stay in registers).
  u32x4 kreg[Tile::CHUNKS], vreg[Tile::CHUNKS];
  const int st_row = tid / (D / 8), st_cc = tid % (D / 8);
  constexpr int ROWS_PER_PASS = 256 / (D / 8);
  const __bf16* const kg = kp + (int64_t)st_row * a.ks.s + st_cc * 8;
  const __bf16* const vg = vp + (int64_t)st_row * a.vs.s + st_cc * 8;
  char* const k_st = k_lds + st_row * Tile::STRIDE + st_cc * 16;
  char* const v_st = v_lds + st_row * Tile::STRIDE + st_cc * 16;
#define AXL_LOAD_TILE(T_)                                                                       \
  _Pragma("unroll") for (int i = 0; i < Tile::CHUNKS; i++) {                                    \
    const int64_t row_ = (int64_t)(T_) * Tile::BK + i * ROWS_PER_PASS;                          \
    kreg[i] = *(const u32x4*)(kg + row_ * a.ks.s);                                              \
    vreg[i] = *(const u32x4*)(vg + row_ * a.vs.s);                                              \
  }
#define AXL_STORE_TILE(BUF_)                                                                    \
  _Pragma("unroll") for (int i = 0; i < Tile::CHUNKS; i++) {                                    \
    *(u32x4*)(k_st + (BUF_) * Tile::TILE_BYTES + i * ROWS_PER_PASS * Tile::STRIDE) = kreg[i];   \
    *(u32x4*)(v_st + (BUF_) * Tile::TILE_BYTES + i * ROWS_PER_PASS * Tile::STRIDE) = vreg[i];   \
  }
  // AUX: raw bias words and dropout bytes of the lane's 4 runs of 8 keys of a tile (run i = keys
  // 32(i/2) + 16(i%2) + 8g .. +7; an fp32 bias fills both vectors of a run, a bf16 bias repeats its one
  // load), requested one tile ahead, together with that tile's K / V rows.  The presence tests are
  // on the arguments, which are uniform (the row pointers differ by lane).
  const bool has_bias = AUX && a.aux.bias != nullptr, has_drop = AUX && a.aux.drop != nullptr;
  const int bias_shift = a.aux.bias_f32 ? 2 : 1, bias_second = a.aux.bias_f32 ? 16 : 0;
  u32x4 bias_nx[AUX ? 8 : 1], bias_cur[AUX ? 8 : 1];
  uint2 drop_nx[AUX ? 4 : 1], drop_cur[AUX ? 4 : 1];
  auto aux_request = [&](int t) __attribute__((always_inline)) {
    if constexpr (AUX) {
      const int key0 = t * Tile::BK + 8 * g;
      if (has_bias) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const char* p = bias_row + ((int64_t)(key0 + 32 * (i / 2) + 16 * (i % 2)) << bias_shift);
          bias_nx[2 * i] = *(const u32x4*)p;
          bias_nx[2 * i + 1] = *(const u32x4*)(p + bias_second);
        }
      }
      if (has_drop) {
#pragma unroll
        for (int i = 0; i < 4; i++) drop_nx[i] = *(const uint2*)(drop_row + key0 + 32 * (i / 2) + 16 * (i % 2));
      }
    }
  };
  auto aux_rotate = [&]() __attribute__((always_inline)) {
    if constexpr (AUX) {
#pragma unroll
      for (int i = 0; i < 8; i++) bias_cur[i] = bias_nx[i];
#pragma unroll
      for (int i = 0; i < 4; i++) drop_cur[i] = drop_nx[i];
    }
  };
  if (t_begin < t_end) {
    AXL_LOAD_TILE(t_begin)
    aux_request(t_begin);
    AXL_STORE_TILE(0)
    aux_rotate();
  }
  wait_all_vmem();  // stationary fragments have landed: nothing issued before the loop is pending
  __syncthreads();

  const int a_row_off = swap_bits_2_3(l32) * Tile::STRIDE + g * 16;
  const int j16 = lane & 15, half = (lane >> 4) & 1;
  const int tr_off = (8 * g + (j16 >> 2)) * Tile::STRIDE + (16 * half + 4 * (j16 & 3)) * 2;

  for (int t = t_begin; t < t_end; t++) {
    const int buf = (t - t_begin) & 1;
    const bool has_next = t + 1 < t_end;
    if (has_next) {
      AXL_LOAD_TILE(t + 1)
      aux_request(t + 1);
    }
    const int k0 = t * Tile::BK;
    bool skip = false, need_mask = false;
    if (a.mask_kind != AXL_MASK_NONE) {
      skip = k0 > qpos_max;
      need_mask = k0 + Tile::BK - 1 > qpos_min;
      if (a.mask_kind == AXL_MASK_SLIDING_WINDOW) {
        skip = skip || (qpos_min - (k0 + Tile::BK - 1) > a.window);
        need_mask = need_mask || (qpos_max - k0 > a.window);
      }
    }
    if (!skip) {
      const char* kt = k_lds + buf * Tile::TILE_BYTES;
      const char* vt = v_lds + buf * Tile::TILE_BYTES;
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        floatx16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
        const char* ka = kt + ks * 32 * Tile::STRIDE + a_row_off;
        const char* va = vt + ks * 32 * Tile::STRIDE + a_row_off;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
          const bf16x8 kfr = *(const bf16x8*)(ka + kk * 32);
          s = E::mfma_32x32x16(kfr, qf[kk], s);
        }
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
          const bf16x8 vfr = *(const bf16x8*)(va + kk * 32);
          dp = E::mfma_32x32x16(vfr, dof[kk], dp);
        }
        // Register r of lane group g is key k0 + 32ks + 16(r/8) + 8g + (r%8); the lane is a query.
        if constexpr (AUX) {
          // logits = scale * qk + bias, kept in raw units as qk + bias / scale; a dropped element
          // has dP = 0, a kept one dP / (1 - rate) (gpu_attention.py:601-603).
          if (has_bias) {
#pragma unroll
            for (int t8 = 0; t8 < 2; t8++) {
              const u32x4 w0 = bias_cur[2 * (2 * ks + t8)], w1 = bias_cur[2 * (2 * ks + t8) + 1];
              float bv[8];
              if (a.aux.bias_f32) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                  const unsigned lo = w0[j], hi = w1[j];
                  bv[j] = __builtin_bit_cast(float, lo);
                  bv[4 + j] = __builtin_bit_cast(float, hi);
                }
              } else {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                  bv[2 * j] = __builtin_bit_cast(float, w0[j] << 16);
                  bv[2 * j + 1] = __builtin_bit_cast(float, w0[j] & 0xffff0000u);
                }
              }
#pragma unroll
              for (int j = 0; j < 8; j++) s[8 * t8 + j] = __builtin_fmaf(bv[j], a.aux.inv_scale, s[8 * t8 + j]);
            }
          }
          if (has_drop) {
#pragma unroll
            for (int t8 = 0; t8 < 2; t8++) {
              const uint2 w = drop_cur[2 * ks + t8];
#pragma unroll
              for (int j = 0; j < 8; j++) {
                const unsigned byte = ((j < 4 ? w.x : w.y) >> (8 * (j % 4))) & 0xffu;
                dp[8 * t8 + j] = byte ? 0.f : dp[8 * t8 + j] * a.aux.keep_scale;
              }
            }
          }
        }
        // Masks in (at most) two wave-uniform blocks; unmasked tiles run straight-line code.
        if (need_mask) {
          const int diff0 = qpos - (k0 + 32 * ks + 8 * g);
          const unsigned limit = a.mask_kind == AXL_MASK_SLIDING_WINDOW ? (unsigned)a.window : 0x7fffffffu;
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const unsigned diff = (unsigned)(diff0 - (16 * (r / 8) + (r % 8)));
            s[r] = diff <= limit ? s[r] : kMasked;  // 0 <= q - k <= limit
          }
        }
        if (seg_k) {
          intx4 seg_v[4];
#pragma unroll
          for (int t8 = 0; t8 < 2; t8++) {
            const intx4* sp = (const intx4*)(seg_k + k0 + 32 * ks + 16 * t8 + 8 * g);
            seg_v[2 * t8] = sp[0];
            seg_v[2 * t8 + 1] = sp[1];
          }
#pragma unroll
          for (int r = 0; r < 16; r++) s[r] = seg_v[r / 4][r % 4] == seg_q ? s[r] : kMasked;
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float p = fast_exp2(__builtin_fmaf(s[r], c, -lse2));
          dp[r] = p * (dp[r] - delta);
        }
        // dQ^T[d][q] += K^T[d][key] dS^T[key][q].
#pragma unroll
        for (int t8 = 0; t8 < 2; t8++) {
          const bf16x8 dsb = pack8<E>(dp[8 * t8 + 0], dp[8 * t8 + 1], dp[8 * t8 + 2], dp[8 * t8 + 3],
                                         dp[8 * t8 + 4], dp[8 * t8 + 5], dp[8 * t8 + 6], dp[8 * t8 + 7]);
          const char* kta = kt + (32 * ks + 16 * t8) * Tile::STRIDE + tr_off;
#pragma unroll
          for (int dt = 0; dt < DT; dt++) {
            union { bf16x8 v; shortx4 hlf[2]; } fa;
            fa.hlf[0] = lds_read_tr16(kta + dt * 64);
            fa.hlf[1] = lds_read_tr16(kta + dt * 64 + 4 * Tile::STRIDE);
            dq_acc[dt] = E::mfma_32x32x16(fa.v, dsb, dq_acc[dt]);
          }
        }
      }
    }
    if (has_next) {
      AXL_STORE_TILE(buf ^ 1)
      aux_rotate();
    }
    __syncthreads();
  }
#undef AXL_LOAD_TILE
#undef AXL_STORE_TILE

  __bf16* dqp =(__bf16*)a.dq + b * a.dqs.b + (int64_t)(q0 + l32) * a.dqs.s + h * a.dqs.h;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int rq = 0; rq < 4; rq++) {
      union { bf16x2 p[2]; uint2 u; } w;
      w.p[0] = E::pack(dq_acc[dt][4 * rq + 0] * a.scale, dq_acc[dt][4 * rq + 1] * a.scale);
      w.p[1] = E::pack(dq_acc[dt][4 * rq + 2] * a.scale, dq_acc[dt][4 * rq + 3] * a.scale);
      *(uint2*)(dqp + 32 * dt + 8 * rq + 4 * g) = w.u;
    }
}

// Smallest and largest segment id of every group of 32 consecutive rows ([B, T / 32] groups in all):
// what the dQ and dK/dV kernels classify their loop ranges from (classify_segment_groups_tbl).  One
// thread per group.
__global__ __launch_bounds__(256) void seg_group_table_kernel(const int32_t* seg, int2* tbl, int groups) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= groups) return;
  const intx4* p = (const intx4*)(seg + (int64_t)i * kSegGroupRows);
  int mn = 0x7fffffff, mx = -0x7fffffff - 1;
#pragma unroll
  for (int v = 0; v < kSegGroupRows / 4; v++) {
    const intx4 x = p[v];
    mn = min(min(mn, min(x[0], x[1])), min(x[2], x[3]));
    mx = max(max(mx, max(x[0], x[1])), max(x[2], x[3]));
  }
  tbl[i] = make_int2(mn, mx);
}

static Strides3 to_s3(const AxlStrides& s) { return Strides3{s.batch, s.seq, s.head}; }

// delta and lse2, [B, Hq, T] fp32 each, rounded up to 256 bytes.
static size_t stats_bytes(const AxlFlashBwdParams& p) {
  return (2 * (size_t)p.batch * p.num_q_heads * p.q_len * sizeof(float) + 255) & ~(size_t)255;
}

// The dS-spill path: the dK/dV kernel stores dS and the dQ kernel becomes one streaming GEMM
// (5 executed GEMMs instead of 7).  Causal or sliding-window attention over equal lengths, with or
// without segment ids.
static bool spill_ranged(const AxlFlashBwdParams& p) {
  return p.mask_kind == AXL_MASK_SLIDING_WINDOW || p.segment_ids;
}
static bool spill_eligible(const AxlFlashBwdParams& p) {
  return (p.dtype == AXL_BF16 || p.dtype == AXL_F16) &&
         (p.mask_kind == AXL_MASK_CAUSAL || p.mask_kind == AXL_MASK_SLIDING_WINDOW) && p.q_pos_offset == 0 &&
         p.q_len == p.kv_len && !p.aux.bias && !p.aux.dropout_mask && (p.flags & AXL_BWD_DS_WORKSPACE) &&
         // the ranged kernel keeps the table in LDS beside its ring: 256-row blocks at head_dim 128
         (!spill_ranged(p) || (p.kv_len / 128 <= kMaxKbRanged && (p.head_dim <= 64 || p.q_len % 256 == 0)));
}

// kv heads whose dS the workspace holds at a time (AXL_BWD_DS_SLICE_KV_HEADS in the flags; all of them
// by default): the dK/dV and dQ kernels of the path run once per slice of that many kv heads.
static int spill_slice_heads(const AxlFlashBwdParams& p) {
  const int n = (p.flags >> 8) & 0xffff;
  return n > 0 && n < p.num_kv_heads ? n : p.num_kv_heads;
}
static size_t spill_bytes(const AxlFlashBwdParams& p) {
  const int heads = spill_slice_heads(p) * (p.num_q_heads / p.num_kv_heads);
  return (size_t)p.batch * heads * (size_t)ds_blocks_per_head(p.q_len) * kDsBlockBytes;
}

// With segment ids: the table of per-group id ranges (seg_group_table_kernel), 256-byte rounded.
static size_t seg_table_bytes(const AxlFlashBwdParams& p) {
  if (!p.segment_ids) return 0;
  return ((size_t)p.batch * (p.q_len / kSegGroupRows) * sizeof(int2) + 255) & ~(size_t)255;
}

// Spill path under a sliding window or with segment ids: the query tiles each key block stored dS for.
static size_t kb_table_bytes(const AxlFlashBwdParams& p) {
  if (!spill_eligible(p) || !spill_ranged(p)) return 0;
  return ((size_t)p.batch * (p.kv_len / 128) * sizeof(int2) + 255) & ~(size_t)255;
}

// The parts of the workspace start on 256-byte boundaries; the caller's pointer only has to be
// 16-byte aligned (allocators that slice one arena, XLA's buffer assignment among them, promise less
// than 256), so the size includes the slack for rounding it up.
constexpr size_t kWsAlign = 256;
size_t flash_bwd_workspace_bytes(const AxlFlashBwdParams& p) {
  return stats_bytes(p) + seg_table_bytes(p) + kb_table_bytes(p) + (spill_eligible(p) ? spill_bytes(p) : 0) +
         (kWsAlign - 16);
}

int launch_flash_bwd(const AxlFlashBwdParams& p, int phases, hipStream_t stream) {
  const int dt = p.dtype;
  BwdArgs a;
  a.q = p.q; a.k = p.k; a.v = p.v; a.out = p.out; a.dout = p.d_out; a.lse = p.lse;
  char* const ws = (char*)((reinterpret_cast<uintptr_t>(p.workspace) + (kWsAlign - 1)) & ~(uintptr_t)(kWsAlign - 1));
  a.ndelta = (float*)ws;
  a.lse2 = a.ndelta + (size_t)p.batch * p.num_q_heads * p.q_len;
  a.dq = p.dq; a.dk = p.dk; a.dv = p.dv; a.seg = p.segment_ids;
  const bool spill = spill_eligible(p);  // the entry point has checked that the workspace holds dS as well
  a.seg_tbl = p.segment_ids ? (const int2*)(ws + stats_bytes(p)) : nullptr;
  a.kb_tbl = kb_table_bytes(p) ? (int2*)(ws + stats_bytes(p) + seg_table_bytes(p)) : nullptr;
  a.ds = spill ? ws + stats_bytes(p) + seg_table_bytes(p) + kb_table_bytes(p) : nullptr;
  a.qs = to_s3(p.q_strides); a.ks = to_s3(p.k_strides); a.vs = to_s3(p.v_strides);
  a.os = to_s3(p.out_strides); a.dos = to_s3(p.d_out_strides); a.dqs = to_s3(p.dq_strides);
  a.dks = to_s3(p.dk_strides); a.dvs = to_s3(p.dv_strides);
  a.B = p.batch; a.T = p.q_len; a.S = p.kv_len; a.Hq = p.num_q_heads; a.Hkv = p.num_kv_heads;
  a.mask_kind = p.mask_kind; a.window = p.sliding_window; a.q_off = p.q_pos_offset;
  a.scale = p.softmax_scale;
  a.d_real = p.head_dim;
  a.stat_hq = p.num_q_heads;
  {
    // Two key blocks per dK/dV workgroup under a causal mask, where a block and its mirror image see
    // complementary shares of the queries (an even number of blocks); AXL_DKDV_KB_PER_WG=1 in the
    // environment (read once) keeps one block per workgroup.
    static const bool single = [] { const char* e = getenv("AXL_DKDV_KB_PER_WG"); return e && e[0] == '1'; }();
    a.kb_per_wg = (!single && p.mask_kind == AXL_MASK_CAUSAL && (p.kv_len / 128) % 2 == 0) ? 2 : 1;
  }
  const int width = p.head_dim <= 64 ? 64 : 128;   // the compiled width that serves this head_dim
  a.aux = make_aux_args(p.aux, p.softmax_scale);
  const bool aux = p.aux.bias || p.aux.dropout_mask;
  hipError_t err = hipSuccess;
  const int64_t rows = (int64_t)p.batch * p.q_len * p.num_q_heads;
  const int delta_grid = (int)((rows + 15) / 16);
  const int dkv_grid = (p.kv_len / 128) * p.batch * p.num_kv_heads;
  const int dq_grid = (p.q_len / 128) * p.batch * p.num_q_heads;
#define AXL_LAUNCH(KERNEL, GRID, LDS)                                                           \
  do {                                                                                          \
    if (err == hipSuccess && (LDS) > 0)                                                         \
      err = allow_dynamic_lds((const void*)KERNEL, (LDS));                                      \
    if (err == hipSuccess) {                                                                    \
      hipLaunchKernelGGL(KERNEL, dim3(GRID), dim3(256), (LDS), stream, a);                      \
      err = hipGetLastError();                                                                  \
    }                                                                                           \
  } while (0)
  // All three phases in one call, no bias / dropout mask / sink gradient: the dQ kernel computes delta
  // on the way (it holds the dO rows anyway) and runs first; the dK/dV kernel reads what it left.
  const int all = AXL_BWD_DELTA | AXL_BWD_DKDV | AXL_BWD_DQ;
  if (a.seg_tbl && dt != AXL_F32 && (phases & (AXL_BWD_DKDV | AXL_BWD_DQ))) {
    // every call fills the table it reads: the phases may be enqueued one by one on a fresh workspace
    const int groups = p.batch * (p.q_len / kSegGroupRows);
    hipLaunchKernelGGL(seg_group_table_kernel, dim3((groups + 255) / 256), dim3(256), 0, stream, p.segment_ids,
                       (int2*)a.seg_tbl, groups);
    err = hipGetLastError();
  }
  if (dt == AXL_F32) {
    if (phases & AXL_BWD_DELTA) {
      if (width == 128) AXL_LAUNCH((bwd_delta_kernel<float, 128>), delta_grid, 0);
      else AXL_LAUNCH((bwd_delta_kernel<float, 64>), delta_grid, 0);
    }
    if (err == hipSuccess) err = launch_bwd_f32(a, width, phases, stream);
  } else if (spill) {
    // delta, then the dK/dV kernel (which leaves dS behind), then dq = scale * dS k.
    if (spill_slice_heads(p) < p.num_kv_heads && (phases & AXL_BWD_DKDV) != 0 && (phases & AXL_BWD_DQ) == 0)
      return set_error(AXL_ERR_UNSUPPORTED,
                       "axl_flash_bwd_phases: with dS slices (AXL_BWD_DS_SLICE_KV_HEADS) a slice's dS lives only "
                       "until the next slice's dK/dV kernel: run the DKDV and DQ phases in one call");
    if (phases & AXL_BWD_DELTA) {
      if (dt == AXL_BF16) {
        if (width == 128) AXL_LAUNCH((bwd_delta_kernel<__bf16, 128>), delta_grid, 0);
        else AXL_LAUNCH((bwd_delta_kernel<__bf16, 64>), delta_grid, 0);
      } else {
        if (width == 128) AXL_LAUNCH((bwd_delta_kernel<_Float16, 128>), delta_grid, 0);
        else AXL_LAUNCH((bwd_delta_kernel<_Float16, 64>), delta_grid, 0);
      }
    }
    // One slice of kv heads after the other: the kernels see a problem of that many heads (tensors
    // and statistics offset to the slice's first head) and the same dS workspace.
    const int slice = spill_slice_heads(p), G = p.num_q_heads / p.num_kv_heads, es = 2;
    for (int h0 = 0; h0 < p.num_kv_heads && err == hipSuccess; h0 += slice) {
      BwdArgs s = a;
      s.Hkv = min(slice, p.num_kv_heads - h0);
      s.Hq = s.Hkv * G;
      const int64_t hq0 = (int64_t)h0 * G;
      s.q = (const char*)a.q + hq0 * a.qs.h * es;
      s.dout = (const char*)a.dout + hq0 * a.dos.h * es;
      s.dq = (char*)a.dq + hq0 * a.dqs.h * es;
      s.k = (const char*)a.k + h0 * a.ks.h * es;
      s.v = (const char*)a.v + h0 * a.vs.h * es;
      s.dk = (char*)a.dk + h0 * a.dks.h * es;
      s.dv = (char*)a.dv + h0 * a.dvs.h * es;
      s.ndelta = a.ndelta + hq0 * p.q_len;
      s.lse2 = a.lse2 + hq0 * p.q_len;
      if (phases & AXL_BWD_DKDV) err = launch_bwd_dkdv(s, dt, width, false, stream);
      if ((phases & AXL_BWD_DQ) && err == hipSuccess) err = launch_bwd_dq_stream(s, dt, width, stream);
    }
    phases &= AXL_BWD_DELTA;  // what is left for the code below: the sink gradient
    phases = (phases & AXL_BWD_DELTA) && p.d_logit_sink ? AXL_BWD_DELTA : 0;
    if (phases) {
      hipLaunchKernelGGL(bwd_dsink_kernel, dim3(p.num_q_heads), dim3(256), 0, stream, p.logit_sink,
                         p.lse, a.ndelta, p.d_logit_sink, p.batch, p.num_q_heads, p.q_len);
      if (err == hipSuccess) err = hipGetLastError();
    }
    if (err != hipSuccess)
      return set_error(AXL_ERR_LAUNCH, "axl_flash_bwd: launch failed: %s", hipGetErrorString(err));
    return AXL_OK;
  } else if ((phases & all) == all && !aux && !p.d_logit_sink) {
    err = launch_bwd_dq(a, dt, width, true, stream);
    if (err == hipSuccess) err = launch_bwd_dkdv(a, dt, width, false, stream);
    if (err != hipSuccess)
      return set_error(AXL_ERR_LAUNCH, "axl_flash_bwd: launch failed: %s", hipGetErrorString(err));
    return AXL_OK;
  }
#define AXL_BWD_PHASES(E, T, DD)                                                                  \
  do {                                                                                            \
    if (phases & AXL_BWD_DELTA) AXL_LAUNCH((bwd_delta_kernel<T, DD>), delta_grid, 0);             \
    if ((phases & AXL_BWD_DKDV) && err == hipSuccess) err = launch_bwd_dkdv(a, dt, DD, aux, stream); \
    if ((phases & AXL_BWD_DQ) && aux)                                                             \
      AXL_LAUNCH((flash_bwd_dq_aux_kernel<E, DD, true>), dq_grid, DqTile<DD>::LDS_BYTES);         \
    if ((phases & AXL_BWD_DQ) && !aux && err == hipSuccess) err = launch_bwd_dq(a, dt, DD, false, stream); \
  } while (0)
  if (dt == AXL_F32) {
    // enqueued above
  } else if (dt == AXL_BF16) {
    if (width == 128) AXL_BWD_PHASES(ElemBf16, __bf16, 128);
    else AXL_BWD_PHASES(ElemBf16, __bf16, 64);
  } else {
    if (width == 128) AXL_BWD_PHASES(ElemF16, _Float16, 128);
    else AXL_BWD_PHASES(ElemF16, _Float16, 64);
  }
#undef AXL_BWD_PHASES
#undef AXL_LAUNCH
  if ((phases & AXL_BWD_DELTA) && p.d_logit_sink && err == hipSuccess) {
    hipLaunchKernelGGL(bwd_dsink_kernel, dim3(p.num_q_heads), dim3(256), 0, stream, p.logit_sink,
                       p.lse, a.ndelta, p.d_logit_sink, p.batch, p.num_q_heads, p.q_len);
    err = hipGetLastError();
  }
  if (err != hipSuccess)
    return set_error(AXL_ERR_LAUNCH, "axl_flash_bwd: launch failed: %s", hipGetErrorString(err));
  return AXL_OK;
}

}  // namespace axl
