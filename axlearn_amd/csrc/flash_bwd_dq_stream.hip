// dQ from stored dS for gfx950: the second half of the "dS spill" backward.
//
// The reference's dQ kernel (axlearn/common/flash_attention/gpu_attention.py:533-616) recomputes
// p and ds for every (query block, key block) pair that the dK/dV kernel (:436-528) has already
// visited, so the pair of kernels executes 7 GEMMs of the same size for 5 distinct ones.  Here the
// dK/dV kernel leaves ds, rounded to the input dtype exactly where the reference rounds it
// (`ds.astype(k.dtype)`, :608), in a workspace, and this kernel only forms
//   dq = scale * ds k
// as one streaming GEMM: no exponentials, no second pass over q, dO and v.  It is bound by reading
// ds once from HBM (T^2 bytes per (batch, head) under a causal mask).
//
// Workspace layout (causal mask, q_pos_offset 0, q_len == kv_len): see ds_run_start in flash_bwd.h.
// Query tile t = 4a + r (32 rows) of a head has a contiguous run of 4(a+1) blocks, one per 32 keys that
// the 128 query rows of block a can see.  A block is 2 KB: [q half 2][key 32][16 queries] in the input
// dtype, i.e. the dK/dV kernel's packed dS operand registers written lane by lane.
//
// Mapping.  A workgroup of NW wavefronts owns 32 NW query rows of one (batch, query head); wavefront w
// owns query tile NW qb + w and the fp32 dQ^T accumulators of its 32 rows.  Per trip of 64 keys the K
// tile (shared, XOR-swizzled) and each wavefront's own 4 KB of ds arrive by direct global->LDS loads
// through a ring of buffers; dQ^T += K^T dS^T with both operands from transposing LDS reads.  The
// kernel issues 2.5 LDS reads and half a tile load per MFMA, each of which holds up the wavefront that
// issues it, so it runs with two wavefronts per SIMD where the shape allows (NW = 8, one workgroup of
// 256 rows per CU, three buffers; a wavefront of the upper 128 rows has two trips more than one of
// the lower 128) and with NW = 4 (five buffers) otherwise.
#include "flash_bwd.h"

namespace axl {

template <int D, int NW>
struct DqStream {
  static constexpr int BQ = 32 * NW;         // query rows per workgroup (32 per wavefront)
  static constexpr int BK = 64;              // keys per trip
  static constexpr int ROWB = D * 2;         // bytes per K row: unpadded, chunks swizzled (tile_swizzle)
  static constexpr int K_BYTES = BK * ROWB;
  static constexpr int DS_WAVE_BYTES = 2 * kDsBlockBytes;          // two 32-key blocks per wavefront per trip
  static constexpr int DS_BASE = K_BYTES;
  static constexpr int BUF_BYTES = K_BYTES + NW * DS_WAVE_BYTES;
  static constexpr int NBUF = NW == 8 ? 3 : 5;
  static constexpr int WROWS = BK / NW;                            // K rows that one wavefront fetches
  static constexpr int RPI = 1024 / ROWB;                          // K rows per direct-to-LDS instruction
  static constexpr int K_DMA_PER_WAVE = WROWS / RPI;
  static constexpr int NLD = K_DMA_PER_WAVE + DS_WAVE_BYTES / 1024;  // loads per wavefront per trip
  static constexpr int LDS_BYTES = NBUF * BUF_BYTES;
};

// RANGED: under a sliding window or with segment ids a key block's dK/dV workgroups store the dS of
// the query tiles [first, end) that a.kb_tbl records for it; the other blocks of the workspace hold
// nothing and are skipped (their loads are pointed at the first block, their MFMAs left out).
template <typename E, int D, int NW, bool RANGED>
__global__ __launch_bounds__(64 * NW) void flash_bwd_dq_stream_kernel(const BwdArgs a) {
  using Tile = DqStream<D, NW>;
  constexpr int DT = D / 32;
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  int qb, b, h;
  decode_block(blockIdx.x, a.T / Tile::BQ, a.B, a.Hq, a.Hkv, 32, qb, b, h);
  const int hk = h / (a.Hq / a.Hkv);
  const int q0 = qb * Tile::BQ + wave * 32;
  const int t_q = NW * qb + wave;            // this wavefront's query tile
  int trips = 2 * ((NW * qb + NW - 1) / 4 + 1);  // 64-key tiles up to and including the last diagonal block
  const int my_trips = __builtin_amdgcn_readfirstlane(2 * (t_q / 4 + 1));  // ... of this wavefront's own 128-row block
  int trip0 = 0;                                 // first 64-key tile that any of the workgroup's query tiles has dS for
  __shared__ int2 s_rng[RANGED ? kMaxKbRanged : 1];
  __shared__ int s_first[RANGED ? NW : 1], s_last[RANGED ? NW : 1];
  if constexpr (RANGED) {
    const int nkb = trips / 2;
    const int2* tbl = a.kb_tbl + (int64_t)b * (a.S / 128);
    int first = 0x7fffffff, last = -1;
    for (int i = tid; i < nkb; i += 64 * NW) {
      const int2 r = tbl[i];
      s_rng[i] = r;
      if (r.x < NW * qb + NW && r.y > NW * qb) {   // [r.x, r.y) meets the workgroup's tiles
        first = min(first, i);
        last = max(last, i);
      }
    }
#pragma unroll
    for (int off = 32; off; off >>= 1) {
      first = min(first, __shfl_xor(first, off));
      last = max(last, __shfl_xor(last, off));
    }
    if (lane == 0) {
      s_first[wave] = first;
      s_last[wave] = last;
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < NW; w++) {
      first = min(first, s_first[w]);
      last = max(last, s_last[w]);
    }
    first = __builtin_amdgcn_readfirstlane(first);
    last = __builtin_amdgcn_readfirstlane(last);
    trip0 = last < 0 ? 0 : 2 * first;
    trips = last < 0 ? 0 : 2 * (last + 1);
  }
  // Does this wavefront's query tile have dS for the key block of 64-key tile `trip`?
  auto has_ds = [&](int trip) __attribute__((always_inline)) {
    if constexpr (RANGED) {
      const int2 r = s_rng[trip >> 1];
      return __builtin_amdgcn_readfirstlane((int)(r.x <= t_q && t_q < r.y)) != 0;
    } else {
      return true;
    }
  };

  floatx16 dq_acc[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq_acc[i][r] = 0.f;

  // ---- tile loads.  K: wavefront w fetches rows 16w .. 16w+15 of the tile, lane l the chunk that the
  // swizzle puts at slot l % CPR of row l / CPR.  dS: the wavefront's own run of blocks, copied verbatim.
  constexpr int CPR = D / 8;
  unsigned k_lane[Tile::K_DMA_PER_WAVE];
#pragma unroll
  for (int i = 0; i < Tile::K_DMA_PER_WAVE; i++) {
    const int row = Tile::WROWS * wave + Tile::RPI * i + lane / CPR;
    const int slot_chunk = (lane % CPR) ^ tile_swizzle<D>(row);
    const int chunk = slot_chunk * 8 < a.d_real ? slot_chunk : 0;
    // the second load of a pair carries an instruction offset of 1024, which also moves its source
    k_lane[i] = (unsigned)(row * (int)a.ks.s + chunk * 8) * 2 - (i % 2) * 1024;
  }
  static_assert(Tile::K_DMA_PER_WAVE % 2 == 0, "K loads are issued in pairs");
  const int64_t k_step = (int64_t)Tile::BK * a.ks.s;
  const __bf16* k_src = (const __bf16*)a.k + b * a.ks.b + hk * a.ks.h + trip0 * k_step;
  const int G = a.Hq / a.Hkv;
  const char* ds_src = (const char*)a.ds + ds_run_start((int64_t)b * a.Hkv + hk, a.T, G, t_q, h - hk * G) * kDsBlockBytes +
                       (int64_t)trip0 * Tile::DS_WAVE_BYTES;
  const unsigned ds_lane = 16 * lane;
  const unsigned lds0 = lds_address(smem);
#define AXL_DMA_TRIP(BUF_)                                                                         \
  {                                                                                               \
    const unsigned kdst_ = lds0 + (BUF_) * Tile::BUF_BYTES + wave * (Tile::WROWS * Tile::ROWB);   \
    _Pragma("unroll") for (int i = 0; i < Tile::K_DMA_PER_WAVE; i += 2)                           \
      dma16x2(k_lane[i], k_lane[i + 1], k_src, kdst_ + i * 1024);                                 \
    const unsigned ddst_ = lds0 + (BUF_) * Tile::BUF_BYTES + Tile::DS_BASE + wave * Tile::DS_WAVE_BYTES; \
    const char* dsrc_ = has_ds(pf) ? ds_src : (const char*)a.ds;                                  \
    _Pragma("unroll") for (int i = 0; i < Tile::DS_WAVE_BYTES / 2048; i++)                        \
      dma16x2(ds_lane, ds_lane, dsrc_ + i * 2048, ddst_ + i * 2048);                              \
  }
  // Prefetch cursor; it stops at the last trip (re-fetching that trip is harmless), the dS part of it
  // at the last trip of this wavefront's own run of blocks.
  int pf = trip0;
#define AXL_ADVANCE()                                                       \
  {                                                                         \
    const bool adv_ = pf + 1 < trips;                                       \
    ds_src += __builtin_amdgcn_readfirstlane(pf + 1 < my_trips ? Tile::DS_WAVE_BYTES : 0); \
    pf += adv_ ? 1 : 0;                                                     \
    k_src += adv_ ? k_step : 0;                                             \
  }

  // ---- per-lane LDS read offsets.  K^T fragments (A operands): transposing reads of the swizzled K
  // tile, row 8g + j16/4 (+4 for the second half, +16 per 16-key group), logical byte column
  // (16 half + 4 (j16 % 4)) * 2 + 64 dt.  dS^T fragments (B operands, lane = query l32, keys 8g .. +7
  // of a 16-key group): transposing reads of a block's [key][16 queries] rows of the lane's query half.
  const int j16 = lane & 15, half = (lane >> 4) & 1;
  const int t_row = 8 * g + (j16 >> 2);
  const int t_col = (16 * half + 4 * (j16 & 3)) * 2;
  const int t_off0 = t_row * Tile::ROWB + (t_col & 15), t_off1 = t_off0 + 4 * Tile::ROWB;
  const int t_xor0 = tile_swizzle<D>(t_row) << 4, t_xor1 = tile_swizzle<D>(t_row + 4) << 4;
  int tb_off[2][DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++) {
    tb_off[0][dt] = t_off0 + (((t_col & ~15) + dt * 64) ^ t_xor0);
    tb_off[1][dt] = t_off1 + (((t_col & ~15) + dt * 64) ^ t_xor1);
  }
  const int ds_off = Tile::DS_BASE + wave * Tile::DS_WAVE_BYTES + half * 1024 + (8 * g + (j16 >> 2)) * 32 + (j16 & 3) * 8;
  union TrFrag {
    bf16x8 v;
    shortx4 hlf[2];
  };

  // Everything the compiler tracks has landed before the first untracked load.
  wait_all_vmem();
  constexpr int PF = Tile::NBUF - 1;   // trips in flight ahead of the one being computed
  AXL_DMA_TRIP(0)
#pragma unroll
  for (int i = 1; i < PF; i++) {
    AXL_ADVANCE()
    AXL_DMA_TRIP(i)
  }
  wait_vmem_le<(PF - 1) * Tile::NLD>();   // trip 0 has landed
  __syncthreads();

  constexpr int NM = 4 * DT;          // MFMAs per trip: (32-key block, 16-key group) x dt
  constexpr int kAhead = 4;
  int buf = 0, buf_pf = PF;         // ring slots of trip t and of trip t + PF
  for (int t = trip0; t < trips; t++) {
    const char* kt = smem + buf * Tile::BUF_BYTES;
    // Trip t + PF into the buffer that trip t-1 was read from (every wavefront passed the barrier after it).
    AXL_ADVANCE()
    AXL_DMA_TRIP(buf_pf)
    buf = buf == Tile::NBUF - 1 ? 0 : buf + 1;
    buf_pf = buf_pf == Tile::NBUF - 1 ? 0 : buf_pf + 1;
    if (t < my_trips && has_ds(t)) {
    TrFrag dsf[4], kfr[NM];
#pragma unroll
    for (int s = 0; s < 4; s++) {     // s = 2 * block + 16-key group
      const char* p_ = kt + ds_off + (s / 2) * kDsBlockBytes + (s % 2) * 512;
      dsf[s].hlf[0] = lds_read_tr16(p_);
      dsf[s].hlf[1] = lds_read_tr16(p_ + 128);
    }
#define AXL_K_READ(N_)                                                                     \
  {                                                                                        \
    const int imm_ = 16 * ((N_) / DT) * Tile::ROWB;                                        \
    kfr[N_].hlf[0] = lds_read_tr16(kt + tb_off[0][(N_) % DT] + imm_);                      \
    kfr[N_].hlf[1] = lds_read_tr16(kt + tb_off[1][(N_) % DT] + imm_);                      \
  }
#pragma unroll
    for (int n = 0; n < kAhead; n++) AXL_K_READ(n)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < NM; n++) {
      if (n + kAhead < NM) AXL_K_READ(n + kAhead)
      dq_acc[n % DT] = E::mfma_32x32x16(kfr[n].v, dsf[n / DT].v, dq_acc[n % DT]);
      __builtin_amdgcn_sched_barrier(0);
    }
#undef AXL_K_READ
    }
    // Trip t+1 has landed once at most the loads of the PF - 1 trips after it are outstanding; after
    // the barrier every wavefront's part of it is visible and nobody reads trip t's buffer any more.
    wait_vmem_le<(PF - 1) * Tile::NLD>();
    __syncthreads();
  }
  // The cursor re-requests the last trip during the final trips; none of those loads may still be in
  // flight when this workgroup's LDS is handed to the next one.
  wait_all_vmem();
#undef AXL_DMA_TRIP
#undef AXL_ADVANCE

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

template <typename E, int D, int NW, bool RANGED>
static hipError_t launch_nw(const BwdArgs& a, hipStream_t stream) {
  using Tile = DqStream<D, NW>;
  auto kernel = flash_bwd_dq_stream_kernel<E, D, NW, RANGED>;
  hipError_t err = allow_dynamic_lds((const void*)kernel, Tile::LDS_BYTES);
  if (err != hipSuccess) return err;
  const int grid = (a.T / Tile::BQ) * a.B * a.Hq;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(64 * NW), Tile::LDS_BYTES, stream, a);
  return hipGetLastError();
}

template <typename E, int D>
static hipError_t launch_one(const BwdArgs& a, hipStream_t stream) {
  // 8 wavefronts need two K loads per wavefront (head_dim 128) and 256-row blocks
  constexpr int NW8 = D == 128 ? 8 : 4;
  if (D == 128 && a.T % 256 == 0)
    return a.kb_tbl ? launch_nw<E, D, NW8, true>(a, stream) : launch_nw<E, D, NW8, false>(a, stream);
  return a.kb_tbl ? launch_nw<E, D, 4, true>(a, stream) : launch_nw<E, D, 4, false>(a, stream);
}

hipError_t launch_bwd_dq_stream(const BwdArgs& a, int dtype, int head_dim, hipStream_t stream) {
  if (dtype == AXL_F16) return head_dim == 128 ? launch_one<ElemF16, 128>(a, stream) : launch_one<ElemF16, 64>(a, stream);
  return head_dim == 128 ? launch_one<ElemBf16, 128>(a, stream) : launch_one<ElemBf16, 64>(a, stream);
}

}  // namespace axl
