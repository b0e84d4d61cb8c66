// Single-token decode attention for gfx950: paged KV pool and contiguous KV cache.
//
// Replaces axlearn/common/flash_attention/gpu_paged_attention.py:38-152 (`_paged_attention_kernel`)
// with its launcher and XLA combine (:164-296), and axlearn/common/flash_attention/
// gpu_decoding.py:71-283 (`_attn_forward_kernel`, `_decode_attn_unbatched`).
//
// The operation is bound by HBM: every K and V byte of the live context is read exactly once.
//   * split-K over the context in blocks of `chunk_pages` logical pages (16 tokens each) of one
//     (sequence, kv head).  The split kernel is persistent (two workgroups of 4 wavefronts per CU):
//     every workgroup derives the list of live blocks from the lengths and draws runs of
//     consecutive blocks from a global counter, long runs first and single blocks at the end, so
//     that blocks past a sequence's length cost nothing and CUs that are served faster by the
//     memory system take more of the work;
//   * K and V pages stream from HBM straight into a private LDS ring per wavefront
//     (global_load_lds), so the bytes in flight cost no registers; a stage is refilled as soon as
//     its fragments sit in registers.  The pages of a run are handed to the 4 wavefronts through a
//     counter in LDS, so they finish together;
//   * per page a wavefront computes S^T = K Q^T (v_mfma_f32_16x16x32_bf16) for all query heads of
//     the kv head (padded to 16 columns) and O^T += V^T P^T (v_mfma_f32_16x16x16_bf16, V^T through
//     transposing LDS reads); the accumulator layout of the first product is the operand layout
//     of the second, so probabilities never leave registers;
//   * each run inside one (sequence, kv head) yields one partial record (o, m, l) in an fp32
//     workspace (the reference stores partial o in the query dtype, gpu_paged_attention.py:272)
//     and a second small kernel merges the records of a (sequence, kv head) in context order.
// Work is handed out by timing, so the grouping of the fp32 partial sums - not the set of keys -
// can differ between two calls; the AXL_DECODE_DETERMINISTIC flag of the call (or
// AXL_DECODE_DETERMINISTIC=1 in the environment, read once, as the default for every call) selects
// a fixed decomposition (one block per record, pages dealt round-robin) whose result is
// reproducible bit for bit.
// Keys at index >= length are masked (gpu_paged_attention.py:100, gpu_decoding.py:109); the query
// position is length-1, so a sliding window w also masks keys with (length-1) - j > w.  A page
// index outside the pool reads as zeros and a negative one counts from the end of the pool, as the
// reference's gather does (kv_cache/paged_kv_cache.py:32).
#include <mutex>

#include "common.h"

namespace axl {

struct DecArgs {
  const __bf16* q;        // [B, Hq, D]
  const __bf16* k;        // paged: [Hkv, P, page_size, D]; contiguous: [B, S, Hkv, D] (strided)
  const __bf16* v;
  const int32_t* page_tables;  // [B, pt_stride] (paged only)
  const int32_t* lengths;      // [B]
  __bf16* out;                 // [B, Hq, D]
  float* ws_o;                 // [records, GP, D]; at most B * Hkv * NCH records
  float* ws_m;                 // [records, GP]
  float* ws_l;                 // [records, GP]
  int32_t* ws_tab;             // [B, Hkv, NCH]: record that starts at this live chunk, or -1; every live
                               // chunk's entry is written by the workgroup that streams the chunk
  Strides3 ks, vs;             // contiguous only
  int B, Hq, Hkv, G;
  int ngrp, Hv;                // groups of 16 query heads per kv head; Hv = Hkv * ngrp "virtual" kv heads:
                               // a kv head with more than 16 query heads is streamed once per group
  int num_pages, pps;          // pool pages; 16-token tiles per sequence (ceil(S/16) if contiguous)
  int page_shift, pt_stride;   // a pool page holds 16 << page_shift tokens; entries per page-table row
  int d_real;                  // head_dim of the tensors (a multiple of 8, <= the compiled width D)
  int kv_len;                  // key positions a sequence can address (cache rows / table capacity)
  const char* bias;            // [B|1, Hq|1, kv_len] additive logit bias, bf16 or fp32, or nullptr
  int64_t bias_sb, bias_sh;    // BYTES per batch / query head (0 broadcasts)
  int bias_f32;
  float inv_scale;             // 1 / scale: the bias joins the raw (unscaled) logits
  int chunk_pages, nch;
  int window;
  float scale;
  int* ticket;                 // [0] blocks handed out: zero when the split kernel starts (zeroed by
                               // decode_plan_kernel, or left at zero by the previous call's combine kernel)
  int deterministic;           // fixed work decomposition: results reproducible bit for bit
  int static_only;             // no more blocks than workgroups: block i goes to workgroup i, the counter is not used
};

// Tokens per tile: the unit the kernels stream and compute on.  A pool page of 16 << page_shift
// tokens is that many consecutive tiles (the reference gathers gpu_block_size / page_size pages per
// compute block, gpu_paged_attention.py:91-94; here the compute block is a tile and a page spans
// several).
constexpr int kPage = 16;

// One element of the bias row of (sequence b, query head h) at key position t, in raw-logit units.
__device__ __forceinline__ float decode_bias_at(const DecArgs& a, int b, int h, int t) {
  const char* row = a.bias + b * a.bias_sb + h * a.bias_sh;
  const float x = a.bias_f32 ? ((const float*)row)[t] : (float)((const __bf16*)row)[t];
  return x * a.inv_scale;
}

// XOR swizzle of the 16-byte chunks of a K row inside an LDS tile, so that 16 lanes reading the
// same logical chunk of 16 different rows hit 16 different bank groups.
template <int D>
__device__ __forceinline__ int k_swizzle(int row) {
  if (D == 128) return ((row & 3) << 2) | ((row >> 2) & 3);
  return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
}

// The same for V rows: the transposing read of a 16-column block touches 32 bytes of 16 rows;
// rows 0..7 (and 8..15) are spread over all banks.
template <int D>
__device__ __forceinline__ int v_swizzle(int row) {
  if (D == 128) return 2 * (row & 7);
  return 2 * ((row >> 1) & 3);
}

// Sequences per launch: bounds the work-item tables each workgroup keeps in LDS.
constexpr int kMaxBatch = 512;

// Live chunk range [ch0, ch1) of a sequence of length `len`.
__device__ __forceinline__ void live_chunks(const DecArgs& a, int len, int& ch0, int& ch1) {
  const int npages = min((len + kPage - 1) / kPage, a.pps);
  const int first_page = a.window >= 0 ? max(0, len - 1 - a.window) / kPage : 0;
  ch0 = first_page / a.chunk_pages;
  ch1 = max(ch0, (npages + a.chunk_pages - 1) / a.chunk_pages);
}

// Lengths outside [0, capacity] are clamped: a sequence cannot hold more keys than its page table
// (or its cache rows) can address, and a non-positive length is an empty context.
__device__ __forceinline__ int clamp_length(const DecArgs& a, int len) {
  return max(0, min(len, a.kv_len));
}

template <int D, int GP, int NST>
struct DecTile {
  static constexpr int ROW_BYTES = D * 2;
  static constexpr int TILE_BYTES = kPage * ROW_BYTES;   // K (or V) of one page
  static constexpr int STAGE_BYTES = 2 * TILE_BYTES;     // K then V
  static constexpr int RING_BYTES = 4 * NST * STAGE_BYTES;
  static constexpr int RED_BYTES = 2 * 4 * 16 * 4;
  static constexpr int RED_BASE = RING_BYTES;
  static constexpr int PFX_BASE = RED_BASE + RED_BYTES;   // int[kMaxBatch + 4]: work-item prefix
  static constexpr int LEN_BASE = PFX_BASE + (kMaxBatch + 4) * 4;  // int[kMaxBatch]: sequence lengths
  static constexpr int NEXT_BASE = LEN_BASE + kMaxBatch * 4;       // int[4]: next run, record index
  static constexpr int LDS_BYTES = NEXT_BASE + 16;
  static constexpr int RED_O_PITCH = D + 4;              // floats per (wave, head) row of the epilogue
  static_assert(4 * GP * RED_O_PITCH * 4 <= RING_BYTES, "epilogue staging must fit in the ring");
};

// Split-K kernel.  Per page a wavefront computes
//   S^T = K Q^T     (v_mfma_f32_16x16x32_bf16, A = K rows from LDS, B = Q^T held in registers),
//   O^T += V^T P^T  (v_mfma_f32_16x16x16_bf16, A = V^T through transposing LDS reads, B = P^T),
// in the "transposed" form where lane l owns query head l%16 and the tokens 4*(l/16)..+3 of the
// page: the accumulator layout of S^T is exactly the B-operand layout of the second product, so
// probabilities never leave registers, and every softmax statistic is per lane.
template <typename E, int D, int GP, bool PAGED, int NST, bool BIAS>
__global__ __launch_bounds__(256) void decode_split_kernel(const DecArgs a) {
  using Tile = DecTile<D, GP, NST>;
  constexpr int KSTEPS = D / 32;        // MFMA k-steps over head_dim for S^T
  constexpr int NB = D / 16;            // 16-row blocks of O^T
  constexpr int SL = D / 8;             // 16-byte slices per token row
  constexpr int TPL = 64 / SL;          // token rows covered by one wave-wide load
  constexpr int NLOAD = kPage / TPL;    // wave-wide loads per K (or V) page
  constexpr int LPP = 2 * NLOAD;        // loads in flight per page
  static_assert(LPP * (NST - 1) <= 63, "vmcnt is 6 bits");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float(*red_o)[Tile::RED_O_PITCH] = (float(*)[Tile::RED_O_PITCH])smem;  // [wave*GP + head][d], aliases the ring
  float(*red_m)[16] = (float(*)[16])(smem + Tile::RED_BASE);
  float(*red_l)[16] = red_m + 4;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  // ---- every workgroup builds the same exclusive prefix of live-block counts over the batch.
  int* pfx = (int*)(smem + Tile::PFX_BASE);
  int* lens = (int*)(smem + Tile::LEN_BASE);
  {
    constexpr int PER = kMaxBatch / 256;  // consecutive sequences per thread
    int cnt[PER], tsum = 0;
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int bi = tid * PER + i;
      int n = 0;
      if (bi < a.B) {
        const int l = clamp_length(a, a.lengths[bi]);
        lens[bi] = l;
        int c0, c1;
        live_chunks(a, l, c0, c1);
        n = c1 - c0;
      }
      cnt[i] = n;
      tsum += n;
    }
    int incl = tsum;  // inclusive scan over the wavefront
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d, 64);
      if (lane >= d) incl += up;
    }
    int* wsum = (int*)(smem + Tile::RED_BASE);
    if (lane == 63) wsum[wave] = incl;
    __syncthreads();
    int run = incl - tsum;
    for (int w = 0; w < wave; w++) run += wsum[w];
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int bi = tid * PER + i;
      if (bi <= a.B) pfx[bi] = run;
      run += cnt[i];
    }
    if (tid == 255) pfx[kMaxBatch] = run;
    __syncthreads();
  }
  // ---- work distribution.  The unit of work is a block of `chunk_pages` pages of one (sequence,
  // kv head); blocks are numbered sequence-major, then kv head, then position.  A workgroup draws
  // runs of consecutive blocks from a global counter - long runs while plenty of work is left,
  // single blocks at the end (guided self-scheduling) - so that workgroups on CUs that get more
  // of the memory system take more of the work.  The part of a run inside one (sequence, kv head)
  // is a segment: one contiguous page range, streamed without a break, one partial record.
  const int n_blocks = pfx[a.B] * a.Hv;
  const int n_wg = gridDim.x;
  // The ids of at most 256 pages are kept in registers.  A fixed decomposition (one block per
  // record, pages dealt round-robin) makes the result independent of timing.
  const int max_run = a.deterministic ? 1 : max(1, 256 / a.chunk_pages);
  const int run0 = min(max_run, max(1, n_blocks / (2 * n_wg)));
  int* s_next = (int*)(smem + Tile::NEXT_BASE);
  int* s_page = s_next + 3;  // next page of the segment to hand to a wavefront
  if (tid == 0) *s_page = 4 * NST;
  __syncthreads();
  int run_e = blockIdx.x * run0;
  int run_end = min(run_e + run0, n_blocks);
  int handed = n_wg * run0;  // estimate of how many blocks have been handed out
  while (run_e < n_blocks) {
  bool first_segment = true;
  int next_e = 0, next_n = 0;
  while (run_e < run_end) {
  int b = 0;
  for (int hi = a.B; hi - b > 1;) {  // last b with Hv * pfx[b] <= run_e
    const int mid = (b + hi) >> 1;
    if (pfx[mid] * a.Hv <= run_e) b = mid; else hi = mid;
  }
  const int len = lens[b];
  int ch0, ch1;
  live_chunks(a, len, ch0, ch1);
  const int rem = run_e - pfx[b] * a.Hv;
  const int hv = rem / (ch1 - ch0), cl = rem % (ch1 - ch0);
  // Virtual head -> kv head and group of (at most) 16 of its query heads.
  const int hk = a.ngrp == 1 ? hv : hv / a.ngrp;
  const int grp = hv - hk * a.ngrp;
  const int gcount = min(16, a.G - 16 * grp);
  const int hbase = hk * a.G + 16 * grp;
  const int seg = min(run_end - run_e, ch1 - ch0 - cl);
  int first_page = 0;
  if (a.window >= 0) first_page = max(0, (len - 1 - a.window)) / kPage;
  const int c_begin = max((ch0 + cl) * a.chunk_pages, first_page);
  const int c_end = min((ch0 + cl + seg) * a.chunk_pages, min((len + kPage - 1) / kPage, a.pps));
  // Pages of the segment are numbered 0 .. n_pg-1.  A wavefront starts with pages wave + 4*i,
  // i < NST, and draws further ones from a counter in LDS whenever a ring stage frees up, so that
  // the 4 wavefronts finish together however unevenly the memory system serves them.
  const int n_pg = c_end - c_begin;

  // Draw the next run; the round trip overlaps the loads of Q and of the page ids below.  The
  // segment's record slot is the number of its first block: unique, and below the B * Hkv * NCH
  // records the workspace holds.
  const int rec = run_e;
  if (tid == 0 && first_segment) {
    next_n = min(max_run, max(1, (n_blocks - handed) / (4 * n_wg)));
    next_e = a.static_only ? n_blocks : atomicAdd(&a.ticket[0], next_n);
  }
  first_segment = false;

  // Q^T as MFMA B operand: lane (head column = lane%16, k-group = lane/16) holds d = 32s + 8kg .. +7.
  const int head = lane & 15, kg = lane >> 4;
  bf16x8 qf[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; s++) {
    if (head < gcount && 32 * s + 8 * kg < a.d_real) {
      qf[s] = *(const bf16x8*)(a.q + ((int64_t)b * a.Hq + hbase + head) * a.d_real + 32 * s + 8 * kg);
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) qf[s][e] = (__bf16)0.f;
    }
  }
  // Pool page of each tile of the segment (at most 256 tiles): register r, lane l holds tile 64r + l.
  int seg_pages[4] = {0, 0, 0, 0};
  if (PAGED) {
#pragma unroll
    for (int r = 0; r < 4; r++)
      if (64 * r + lane < n_pg)
        seg_pages[r] = a.page_tables[(int64_t)b * a.pt_stride + ((c_begin + 64 * r + lane) >> a.page_shift)];
  }
  auto page_id = [&](int idx) -> int {
    int pg = __builtin_amdgcn_readlane(seg_pages[0], idx & 63);
#pragma unroll
    for (int r = 1; r < 4; r++)
      if ((idx >> 6) == r) pg = __builtin_amdgcn_readlane(seg_pages[r], idx & 63);
    if (pg < 0) pg += a.num_pages;  // negative indices count from the end, as in the reference's gather
    return pg;
  };

  const int vslice = lane % SL;       // load layout: 16-byte slice of the row
  const int vtok = lane / SL;         // load layout: token row within a load
  const float c = a.scale * kLog2e;

  float m_run = kNegInf, l_run = 0.f;
  floatx4 o[NB];                      // O^T rows d = 16nb + 4kg + r, column = head
#pragma unroll
  for (int nb = 0; nb < NB; nb++) o[nb] = floatx4{0.f, 0.f, 0.f, 0.f};

  // Per-lane source offsets (elements) of the wave-wide loads of a page, and LDS read offsets.
  // Both tiles are stored with their 16-byte chunks XOR-swizzled by a function of the row, which
  // makes the K reads (16 lanes = 16 rows, same chunk) and the transposing V reads (rows 0..7 of
  // the same 32-byte column window) hit distinct banks.
  const int64_t k_row_stride = PAGED ? a.d_real : a.ks.s;
  const int64_t v_row_stride = PAGED ? a.d_real : a.vs.s;
  // A head_dim below the compiled width: the slices past it are fetched from slice 0 of the same row
  // instead.  Those LDS columns then hold finite copies of real data; the Q columns they meet are
  // zero, and the output rows they produce are never written.
  const int real_slices = a.d_real >> 3;
  int k_src[NLOAD], v_src[NLOAD];
#pragma unroll
  for (int i = 0; i < NLOAD; i++) {
    const int row = TPL * i + vtok;
    const int ksl = vslice ^ k_swizzle<D>(row), vsl = vslice ^ v_swizzle<D>(row);
    k_src[i] = (ksl < real_slices ? ksl : 0) * 8;     // + row * stride, added per page
    v_src[i] = (vsl < real_slices ? vsl : 0) * 8;
  }
  int k_rd[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; s++) k_rd[s] = (lane & 15) * Tile::ROW_BYTES + (((4 * s + kg) ^ k_swizzle<D>(lane & 15)) << 4);
  // Transposing V read for block nb: this lane points at row 4kg + (lane%16)/4, columns
  // 16nb + 4*(lane%4) .. +3, i.e. chunk 2nb + (lane%4)/2, half (lane%4)%2.
  const int vrow = 4 * kg + ((lane & 15) >> 2);
  const int v_rd0 = vrow * Tile::ROW_BYTES + ((lane & 2) << 3) + ((lane & 1) << 3);
  const int v_xor = v_swizzle<D>(vrow) << 4;
  const unsigned ring_lds = lds_address(smem) +
                            wave * (NST * Tile::STAGE_BYTES);
  char* ring = smem + wave * (NST * Tile::STAGE_BYTES);

  // Everything the compiler tracks has landed before the first untracked load is issued.
  wait_all_vmem();

  // Issues the 2*NLOAD loads of page `idx` of the segment into ring stage `st`.
  auto issue = [&](int idx, int st) {
    const int j = c_begin + idx;
    const __bf16 *kb, *vb;
    if (PAGED) {
      int pg = page_id(idx);
      if ((unsigned)pg >= (unsigned)a.num_pages) pg = 0;  // reads as zeros: see `valid` below
      // tile (j mod tiles-per-page) of pool page pg of kv head hk
      const int64_t tile = ((((int64_t)hk * a.num_pages + pg) << a.page_shift) + (j & ((1 << a.page_shift) - 1)));
      const int64_t off = tile * (kPage * a.d_real);
      kb = a.k + off;
      vb = a.v + off;
    } else {
      kb = a.k + b * a.ks.b + hk * a.ks.h;
      vb = a.v + b * a.vs.b + hk * a.vs.h;
    }
    const unsigned dst = __builtin_amdgcn_readfirstlane(ring_lds + st * Tile::STAGE_BYTES);
#pragma unroll
    for (int i = 0; i < NLOAD; i++) {
      // Rows past the end of a contiguous cache are clamped to its last row; they are masked.
      const int row = PAGED ? TPL * i + vtok : min(j * kPage + TPL * i + vtok, a.kv_len - 1);
      dma16(kb + row * k_row_stride + k_src[i], dst + i * 1024);
    }
#pragma unroll
    for (int i = 0; i < NLOAD; i++) {
      const int row = PAGED ? TPL * i + vtok : min(j * kPage + TPL * i + vtok, a.kv_len - 1);
      dma16(vb + row * v_row_stride + v_src[i], dst + Tile::TILE_BYTES + i * 1024);
    }
  };

  int ring_idx[NST];     // page held (or awaited) by each ring stage
  int issued = 0;
#pragma unroll
  for (int i = 0; i < NST; i++) {
    ring_idx[i] = wave + 4 * i;
    if (ring_idx[i] < n_pg) {
      issue(ring_idx[i], i);
      issued++;
    }
  }
  bool exhausted = issued < NST;
  int st = 0;
  for (int consumed = 0; consumed < issued; consumed++) {
    int idx = ring_idx[0];
#pragma unroll
    for (int i = 1; i < NST; i++)
      if (st == i) idx = ring_idx[i];
    const int j = c_begin + idx;
    // Wait for this page; the younger pages stay in flight.
    const int younger = issued - consumed - 1;
    if (NST > 3 && younger == 3) wait_vmem_le<(NST > 3 ? 3 : 0) * LPP>();
    else if (NST > 2 && younger == 2) wait_vmem_le<(NST > 2 ? 2 : 0) * LPP>();
    else if (NST > 1 && younger == 1) wait_vmem_le<(NST > 1 ? 1 : 0) * LPP>();
    else wait_vmem_le<0>();
    bool valid = true;
    if (PAGED) valid = (unsigned)page_id(idx) < (unsigned)a.num_pages;
    const char* kt = ring + st * Tile::STAGE_BYTES;
    const char* vt = kt + Tile::TILE_BYTES;
    bf16x8 kf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) kf[ks] = *(const bf16x8*)(kt + k_rd[ks]);
    shortx4 vf[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) vf[nb] = lds_read_tr16(vt + v_rd0 + ((nb * 32) ^ v_xor));
    // The stage is free as soon as its fragments sit in registers: refill it right away so that
    // the loads of page it+NST overlap the arithmetic of this one.
    wait_lds_reads();
    if (!exhausted) {
      int nxt = idx + 4 * NST;
      if (!a.deterministic) {
        if (lane == 0) nxt = atomicAdd(s_page, 1);
        nxt = __builtin_amdgcn_readfirstlane(nxt);
      }
      if (nxt < n_pg) {
        issue(nxt, st);
#pragma unroll
        for (int i = 0; i < NST; i++)
          if (st == i) ring_idx[i] = nxt;
        issued++;
      } else {
        exhausted = true;
      }
    }
    // ---- scores: S^T[token][head]; this lane: head = lane%16, tokens 4kg + r
    floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) s = E::mfma_16x16x32(kf[ks], qf[ks], s);
    if constexpr (BIAS) {
      // logits = scale * q.k + bias (gpu_decoding.py:117-121, gpu_paged_attention.py:103-106): in raw
      // units, bias / scale.  Positions past the row's end are masked below; their reads are clamped.
      if (head < gcount) {
#pragma unroll
        for (int r = 0; r < 4; r++)
          s[r] += decode_bias_at(a, b, hbase + head, min(j * kPage + 4 * kg + r, a.kv_len - 1));
      }
    }
    // A page that straddles the length (or the window start) holds tokens whose probability is
    // exactly 0; their V rows may be uninitialised pool memory, and 0 * NaN would poison the sum,
    // so those rows are replaced by zeros, as are all rows of a page outside the pool.
    const bool boundary = (j * kPage + kPage > len) || (a.window >= 0 && len - 1 - j * kPage > a.window);
    if (boundary || !valid) {
      if (!valid) s = floatx4{0.f, 0.f, 0.f, 0.f};  // a page outside the pool reads as zeros
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int tpos = j * kPage + 4 * kg + r;
        bool keep = tpos < len;
        if (a.window >= 0) keep = keep && (len - 1 - tpos <= a.window);
        s[r] = keep ? s[r] : kMasked;
        if (!keep || !valid) {
#pragma unroll
          for (int nb = 0; nb < NB; nb++) vf[nb][r] = 0;
        }
      }
    }
    float mx = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(m_run, mx);
    const bool changed = mn != m_run;
    const float corr = fast_exp2((m_run - mn) * c);
    m_run = mn;
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      s[r] = fast_exp2((s[r] - mn) * c);
      psum += s[r];
    }
    l_run = l_run * corr + psum;
    union { shortx4 v; bf16x2 p[2]; } pf;
    pf.p[0] = E::pack(s[0], s[1]);
    pf.p[1] = E::pack(s[2], s[3]);
    if (__builtin_amdgcn_ballot_w64(changed) != 0) {
#pragma unroll
      for (int nb = 0; nb < NB; nb++) o[nb] *= corr;
    }
    // ---- O^T += V^T P^T
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
      o[nb] = E::mfma_16x16x16(vf[nb], pf.v, o[nb]);
    st = (st + 1 == NST) ? 0 : st + 1;
  }

  // ---- merge the 4 wavefronts of this workgroup.
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if (kg == 0) {
    red_m[wave][head] = m_run;
    red_l[wave][head] = l_run;
  }
  __syncthreads();  // also: every wavefront is done with its ring, which red_o aliases
  {
    const float mw = fmaxf(fmaxf(red_m[0][head], red_m[1][head]), fmaxf(red_m[2][head], red_m[3][head]));
    const float f_wave = fast_exp2((m_run - mw) * c);
    if (head < GP) {
#pragma unroll
      for (int nb = 0; nb < NB; nb++)
        *(float4*)&red_o[wave * GP + head][16 * nb + 4 * kg] =
            float4{o[nb][0] * f_wave, o[nb][1] * f_wave, o[nb][2] * f_wave, o[nb][3] * f_wave};
    }
  }
  __syncthreads();
  const int64_t slot = rec;
  float* out_ws = a.ws_o + slot * (GP * D);
  for (int idx = tid; idx < GP * D; idx += 256) {
    const int gq = idx / D, d = idx % D;
    out_ws[idx] = red_o[gq][d] + red_o[GP + gq][d] + red_o[2 * GP + gq][d] + red_o[3 * GP + gq][d];
  }
  if (tid < GP) {
    const float mw = fmaxf(fmaxf(red_m[0][tid], red_m[1][tid]), fmaxf(red_m[2][tid], red_m[3][tid]));
    float lw = 0.f;
#pragma unroll
    for (int w = 0; w < 4; w++) lw += red_l[w][tid] * fast_exp2((red_m[w][tid] - mw) * c);
    a.ws_m[slot * GP + tid] = mw;
    a.ws_l[slot * GP + tid] = lw;
  }
  // Table entries of the segment's chunks: the record at its first chunk, "none" at the others.
  for (int i = tid; i < seg; i += 256) a.ws_tab[((int64_t)b * a.Hv + hv) * a.nch + cl + i] = i == 0 ? (int)slot : -1;
  if (tid == 0) *s_page = 4 * NST;
  __syncthreads();  // the ring (and red_m/red_l) are reused by the next segment
  run_e += seg;
  }  // segments of the run
  if (tid == 0) { s_next[0] = n_wg * run0 + next_e; s_next[1] = next_n; }
  __syncthreads();
  run_e = s_next[0];
  run_end = min(run_e + s_next[1], n_blocks);
  handed = run_e + s_next[1];
  __syncthreads();  // s_next is rewritten at the end of the next run
  }  // runs
}

// Zeroes the work counter ahead of the split kernel when the workspace comes with unknown contents
// (a kernel rather than a memset so that the sequence can be captured into a graph).  A workspace
// that the caller declares reused skips it: the combine kernel leaves the counter at zero.
__global__ __launch_bounds__(64) void decode_plan_kernel(int* ticket) {
  if (threadIdx.x == 0) ticket[0] = 0;
}

// Merges the per-chunk partials of one (sequence, kv head): the "final round of flash"
// (gpu_paged_attention.py:287-296, gpu_decoding.py:277-283).
constexpr int kMaxChunks = 256;  // per sequence; bounds the combine kernel's LDS tables

template <typename E, int D, int GP>
__global__ __launch_bounds__(256) void decode_combine_kernel(const DecArgs a) {
  __shared__ float sm[kMaxChunks * GP];   // record maxima, then rescale factors
  __shared__ float sl[kMaxChunks * GP];   // record sums
  __shared__ int s_raw[kMaxChunks];       // the record table row
  __shared__ int s_list[kMaxChunks];      // records of this (sequence, kv head), in chunk order
  __shared__ int s_count;
  __shared__ float s_max[GP], s_inv[GP];
  __shared__ float4 s_part[256];          // partial sums of the record slices
  const int hv = blockIdx.x, b = blockIdx.y;
  const int hk = hv / a.ngrp, grp = hv - hk * a.ngrp;
  const int gcount = min(16, a.G - 16 * grp);   // query heads of this group
  const int hbase = hk * a.G + 16 * grp;
  const int tid = threadIdx.x;
  const int len = clamp_length(a, a.lengths[b]);
  int ch0, ch1;
  live_chunks(a, len, ch0, ch1);
  const int nc = ch1 - ch0;               // live chunks = upper bound on records of this (b, hk)
  // The split kernel has finished: leave the work counter at zero for the next call on this workspace.
  if (hv == 0 && b == 0 && tid == 0) a.ticket[0] = 0;
  const float c = a.scale * kLog2e;
  // The whole table row in one round trip, then compacted in chunk order by one wavefront.
  s_raw[tid] = tid < nc ? a.ws_tab[((int64_t)b * a.Hv + hv) * a.nch + tid] : -1;
  __syncthreads();
  if (tid < 64) {
    int count = 0;
    for (int base = 0; base < nc; base += 64) {
      const int r = s_raw[base + tid];
      const unsigned long long mask = __builtin_amdgcn_ballot_w64(r >= 0);
      if (r >= 0) s_list[count + __builtin_popcountll(mask & ((1ull << tid) - 1))] = r;
      count += __builtin_popcountll(mask);
    }
    if (tid == 0) s_count = count;
  }
  __syncthreads();
  const int nl = s_count;
  const int n = nl * GP;
  for (int i = tid; i < n; i += 256) {
    const int64_t r = s_list[i / GP];
    sm[i] = a.ws_m[r * GP + i % GP];
    sl[i] = a.ws_l[r * GP + i % GP];
  }
  __syncthreads();
  if (tid < GP) {
    float mw = kNegInf;
    for (int i = tid; i < n; i += GP) mw = fmaxf(mw, sm[i]);
    s_max[tid] = mw;
  }
  __syncthreads();
  for (int i = tid; i < n; i += 256) sm[i] = fast_exp2((sm[i] - s_max[i % GP]) * c);
  __syncthreads();
  if (tid < GP) {
    float l = 0.f;
    for (int i = tid; i < n; i += GP) l += sl[i] * sm[i];
    // An empty context (length 0, or no key inside the window) has no record: the output is zeros,
    // as with the reference's o / (l + eps) (gpu_decoding.py:282, gpu_paged_attention.py:291-293).
    s_inv[tid] = l > 0.f ? 1.f / l : 0.f;
  }
  __syncthreads();
  // Output: G*D floats = n4 groups of four.  With fewer groups than threads the records are dealt
  // to `ways` slices of threads (record ci to slice ci % ways), 16 loads in flight per thread,
  // and the slices' partial sums are added in slice order.
  const int n4 = gcount * D / 4;
  const int per = min(n4, 256);
  const int ways = 256 / per;
  for (int base = 0; base < n4; base += per) {
    const int way = tid / per, col = base + tid % per;
    const bool live = way < ways && col < n4;
    const int gq = live ? (4 * col) / D : 0;
    float4 acc = {0.f, 0.f, 0.f, 0.f};
    if (live) {
#pragma unroll 16
      for (int ci = way; ci < nl; ci += ways) {
        const float4 o = *(const float4*)(a.ws_o + (int64_t)s_list[ci] * (GP * D) + 4 * col);
        const float f = sm[ci * GP + gq];
        acc.x += o.x * f; acc.y += o.y * f; acc.z += o.z * f; acc.w += o.w * f;
      }
    }
    if (base > 0) __syncthreads();  // s_part of the previous pass has been read
    s_part[tid] = acc;
    __syncthreads();
    if (live && way == 0) {
      for (int w = 1; w < ways; w++) {
        const float4 p = s_part[w * per + tid];
        acc.x += p.x; acc.y += p.y; acc.z += p.z; acc.w += p.w;
      }
      const float inv = s_inv[gq];
      const int dcol = 4 * col - gq * D;   // column inside the head: the ones past head_dim are padding
      const int64_t at = ((int64_t)b * a.Hq + hbase + gq) * a.d_real + dcol;
      if (dcol < a.d_real) {
        if constexpr (std::is_same_v<E, ElemF32>) {
          *(float4*)((float*)a.out + at) = float4{acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv};
        } else {
          union { bf16x2 p[2]; uint2 u; } pk;
          pk.p[0] = E::pack(acc.x * inv, acc.y * inv);
          pk.p[1] = E::pack(acc.z * inv, acc.w * inv);
          *(uint2*)(a.out + at) = pk.u;
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// fp32 decode (the reference's decode tests run float32, decoding_test.py:33): plain fp32
// multiply-adds and the accurate exponential, one workgroup per live block of `chunk_pages` pages of
// a (sequence, kv head), a fixed decomposition.  A token row is spread over 16 lanes; each 16-lane
// group keeps a running (m, l, o) per query head over the tokens it visits, the groups are merged at
// the end and leave one record in the same format as the 16-bit kernel's, for the same merge kernel.
// For parity with float32 callers, not for speed.
// ---------------------------------------------------------------------------------------------
template <int D, int GP, bool PAGED>
__global__ __launch_bounds__(256) void decode_split_f32_kernel(const DecArgs a) {
  constexpr int SL = D / 16;  // floats of a row per lane
  __shared__ float q_lds[GP * D];
  __shared__ float red_o[4][GP][D];
  __shared__ float red_m[4][GP], red_l[4][GP];
  const int c = blockIdx.x, hv = blockIdx.y, b = blockIdx.z;
  const int hk = hv / a.ngrp, grp = hv - hk * a.ngrp;
  const int gcount = min(16, a.G - 16 * grp);   // query heads of this group
  const int hbase = hk * a.G + 16 * grp;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, sub = lane >> 4, l16 = lane & 15;
  const int len = clamp_length(a, a.lengths[b]);
  int ch0, ch1;
  live_chunks(a, len, ch0, ch1);
  if (ch0 + c >= ch1) return;
  const int npages = min((len + kPage - 1) / kPage, a.pps);
  const int first_page = a.window >= 0 ? max(0, len - 1 - a.window) / kPage : 0;
  const int p_begin = max((ch0 + c) * a.chunk_pages, first_page);
  const int p_end = min((ch0 + c + 1) * a.chunk_pages, npages);
  const float* qg = (const float*)a.q + ((int64_t)b * a.Hq + hbase) * a.d_real;
  for (int i = tid; i < GP * D; i += 256) {
    const int h = i / D, d = i % D;   // columns past head_dim and heads past the group are zero
    q_lds[i] = (h < gcount && d < a.d_real) ? qg[h * a.d_real + d] : 0.f;
  }
  __syncthreads();

  float m[GP], l[GP], o[GP][SL];
#pragma unroll
  for (int h = 0; h < GP; h++) {
    m[h] = kNegInf;
    l[h] = 0.f;
#pragma unroll
    for (int i = 0; i < SL; i++) o[h][i] = 0.f;
  }
  for (int tok = p_begin * kPage + wave * 4 + sub; tok < p_end * kPage; tok += 16) {
    const float *kr, *vr;
    bool valid = true;
    if (PAGED) {
      const int page_tokens = kPage << a.page_shift;
      int pg = a.page_tables[(int64_t)b * a.pt_stride + tok / page_tokens];
      if (pg < 0) pg += a.num_pages;  // negative indices count from the end, as in the reference's gather
      valid = (unsigned)pg < (unsigned)a.num_pages;  // a page outside the pool reads as zeros
      const int64_t off = (((int64_t)hk * a.num_pages + (valid ? pg : 0)) * page_tokens + tok % page_tokens) * a.d_real;
      kr = (const float*)a.k + off;
      vr = (const float*)a.v + off;
    } else {
      const int row = min(tok, a.kv_len - 1);  // rows past the cache are masked below
      kr = (const float*)a.k + b * a.ks.b + (int64_t)row * a.ks.s + hk * a.ks.h;
      vr = (const float*)a.v + b * a.vs.b + (int64_t)row * a.vs.s + hk * a.vs.h;
    }
    bool keep = tok < len;
    if (a.window >= 0) keep = keep && (len - 1 - tok <= a.window);
    if (!keep) continue;  // uniform over the 16 lanes of the token
    float kx[SL], vx[SL];
#pragma unroll
    for (int i = 0; i < SL; i += 4) {
      const bool in = valid && SL * l16 + i < a.d_real;   // head_dim is a multiple of 8: whole groups of 4
      const float4 x = in ? *(const float4*)(kr + SL * l16 + i) : float4{0.f, 0.f, 0.f, 0.f};
      const float4 y = in ? *(const float4*)(vr + SL * l16 + i) : float4{0.f, 0.f, 0.f, 0.f};
      kx[i] = x.x; kx[i + 1] = x.y; kx[i + 2] = x.z; kx[i + 3] = x.w;
      vx[i] = y.x; vx[i + 1] = y.y; vx[i + 2] = y.z; vx[i + 3] = y.w;
    }
#pragma unroll
    for (int h = 0; h < GP; h++) {
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < SL; i++) dot = __builtin_fmaf(q_lds[h * D + SL * l16 + i], kx[i], dot);
      dot += __shfl_xor(dot, 1, 64);
      dot += __shfl_xor(dot, 2, 64);
      dot += __shfl_xor(dot, 4, 64);
      dot += __shfl_xor(dot, 8, 64);
      if (a.bias && h < gcount) dot += decode_bias_at(a, b, hbase + h, tok);
      const float mn = fmaxf(m[h], dot);
      const float corr = expf((m[h] - mn) * a.scale);
      const float pr = expf((dot - mn) * a.scale);
      m[h] = mn;
      l[h] = l[h] * corr + pr;
#pragma unroll
      for (int i = 0; i < SL; i++) o[h][i] = __builtin_fmaf(pr, vx[i], o[h][i] * corr);
    }
  }
  // ---- merge the four 16-lane groups of the wavefront, then the four wavefronts.
#pragma unroll
  for (int h = 0; h < GP; h++) {
    float mw = fmaxf(m[h], __shfl_xor(m[h], 16, 64));
    mw = fmaxf(mw, __shfl_xor(mw, 32, 64));
    const float f = expf((m[h] - mw) * a.scale);
    float lw = l[h] * f;
    lw += __shfl_xor(lw, 16, 64);
    lw += __shfl_xor(lw, 32, 64);
#pragma unroll
    for (int i = 0; i < SL; i++) {
      float x = o[h][i] * f;
      x += __shfl_xor(x, 16, 64);
      x += __shfl_xor(x, 32, 64);
      if (sub == 0) red_o[wave][h][SL * l16 + i] = x;
    }
    if (lane == 0) {
      red_m[wave][h] = mw;
      red_l[wave][h] = lw;
    }
  }
  __syncthreads();
  const int64_t rec = ((int64_t)b * a.Hv + hv) * a.nch + c;
  for (int idx = tid; idx < GP * D; idx += 256) {
    const int h = idx / D, d = idx % D;
    const float mw = fmaxf(fmaxf(red_m[0][h], red_m[1][h]), fmaxf(red_m[2][h], red_m[3][h]));
    float acc = 0.f;
#pragma unroll
    for (int w = 0; w < 4; w++) acc += red_o[w][h][d] * expf((red_m[w][h] - mw) * a.scale);
    a.ws_o[rec * (GP * D) + idx] = acc;
  }
  if (tid < GP) {
    const float mw = fmaxf(fmaxf(red_m[0][tid], red_m[1][tid]), fmaxf(red_m[2][tid], red_m[3][tid]));
    float lw = 0.f;
#pragma unroll
    for (int w = 0; w < 4; w++) lw += red_l[w][tid] * expf((red_m[w][tid] - mw) * a.scale);
    a.ws_m[rec * GP + tid] = mw;
    a.ws_l[rec * GP + tid] = lw;
    if (tid == 0) a.ws_tab[rec] = (int)rec;
  }
}

// Ring depth (pages in flight per wavefront).  head_dim 128: 2 x 8 KB per wavefront, 69 KB per
// workgroup, two workgroups per CU.
constexpr int kStages128 = 2;
constexpr int kStages64 = 4;

// Workgroups the split kernel keeps resident on the GPU it is tuned for (two on each of 256 CUs).
constexpr int kSplitSlots = 512;

// Pages per block of work.  `rows` = (sequence, kv head group) pairs of the call.
static int pick_chunk_pages(int pps, int64_t rows) {
  // 32 pages = 512 tokens = 256 KB of K+V per workgroup at head_dim 128.
  int cp = 32;
  // A small call (one sequence, a short context) has fewer such blocks than the GPU has workgroup slots
  // and is bound by the latency of a block's few rounds of loads: shorter blocks, about one per slot,
  // down to 8 pages (one round of the four wavefronts' rings).
  if (rows > 0 && rows * ((pps + cp - 1) / cp) < kSplitSlots) {
    const int64_t per_row = kSplitSlots / rows;
    cp = (int)(((pps + per_row - 1) / per_row + 3) / 4 * 4);
    cp = cp < 8 ? 8 : (cp > 32 ? 32 : cp);
  }
  if (pps < cp) cp = ((pps + 3) / 4) * 4;
  if (pps > cp * kMaxChunks) cp = ((pps + kMaxChunks - 1) / kMaxChunks + 3) / 4 * 4;
  return cp < 4 ? 4 : cp;
}

constexpr int kWsHeaderFloats = 64;  // 256 bytes ahead of the records: the work counter

static size_t ws_bytes(int B, int Hkv, int nch, int gp, int D) {
  return (size_t)B * Hkv * nch * ((size_t)gp * D + 2 * gp + 1) * sizeof(float) + kWsHeaderFloats * sizeof(float);
}

// Query-head columns a record holds: the heads of a group padded to 4 / 8 / 16.  The kernels that add
// a bias are compiled for 16 only.
static int gp_of(int G, bool bias) { return bias || G > 8 ? 16 : (G <= 4 ? 4 : 8); }
// Groups of at most 16 query heads per kv head ("virtual" kv heads per kv head).
static int groups_of(int G) { return (G + 15) / 16; }
// Compiled head_dim width that serves a head_dim (a multiple of 8, at most 128).
static int width_of(int d) { return d <= 64 ? 64 : 128; }
// log2(page_size / 16), or -1 if the page size is not 16 times a power of two.
static int page_shift_of(int page_size) {
  for (int sh = 0; sh < 16; sh++)
    if (page_size == (kPage << sh)) return sh;
  return -1;
}

static size_t ws_bytes_for(int batch, int hq, int hkv, int d, int tiles, bool bias) {
  const int G = hq / hkv;
  const int cp = pick_chunk_pages(tiles, (int64_t)batch * hkv * groups_of(G));
  const int nch = (tiles + cp - 1) / cp;
  return ws_bytes(batch, hkv * groups_of(G), nch, gp_of(G, bias), width_of(d));
}

size_t paged_decode_workspace_bytes(const AxlPagedDecodeParams& p) {
  const int sh = page_shift_of(p.page_size);
  if (p.pages_per_seq <= 0 || p.num_kv_heads <= 0 || p.num_q_heads < p.num_kv_heads || sh < 0) return 0;
  return ws_bytes_for(p.batch, p.num_q_heads, p.num_kv_heads, p.head_dim, p.pages_per_seq << sh, p.bias.bias != nullptr);
}

size_t decode_workspace_bytes(const AxlDecodeParams& p) {
  if (p.kv_len <= 0 || p.num_kv_heads <= 0 || p.num_q_heads < p.num_kv_heads) return 0;
  return ws_bytes_for(p.batch, p.num_q_heads, p.num_kv_heads, p.head_dim, (p.kv_len + kPage - 1) / kPage,
                      p.bias.bias != nullptr);
}

static void set_bias(DecArgs& a, const AxlDecodeBias& x, float scale) {
  const int es = x.dtype == AXL_F32 ? 4 : 2;
  a.bias = (const char*)x.bias;
  a.bias_sb = x.batch_stride * es;
  a.bias_sh = x.head_stride * es;
  a.bias_f32 = x.dtype == AXL_F32;
  a.inv_scale = 1.0f / scale;
}

// AXL_DECODE_DETERMINISTIC in the environment, read once: the default for calls that do not set the flag.
static bool deterministic_by_default() {
  static const bool v = [] {
    const char* det = getenv("AXL_DECODE_DETERMINISTIC");
    return det && det[0] != '\0' && det[0] != '0';
  }();
  return v;
}

template <typename E, bool PAGED>
static int launch_common(DecArgs a, int flags, hipStream_t stream, const char* who) {
  const int D = width_of(a.d_real);
  const bool bias = a.bias != nullptr;
  const int gp = gp_of(a.G, bias);
  a.ngrp = groups_of(a.G);
  a.Hv = a.Hkv * a.ngrp;
  a.chunk_pages = pick_chunk_pages(a.pps, (int64_t)a.B * a.Hv);
  if (a.chunk_pages > 256)
    return set_error(AXL_ERR_UNSUPPORTED, "%s: context longer than %d tokens", who, 256 * kMaxChunks * kPage);
  a.nch = (a.pps + a.chunk_pages - 1) / a.chunk_pages;
  // Workspace: a 256-byte header (the work counter, at the same place whatever the shapes), then the
  // records, their statistics and the record table.
  a.ticket = (int*)a.ws_o;
  a.ws_o += kWsHeaderFloats;
  float* ws = a.ws_o;
  const size_t n_o = (size_t)a.B * a.Hv * a.nch * gp * D;
  const size_t n_s = (size_t)a.B * a.Hv * a.nch * gp;
  a.ws_m = ws + n_o;
  a.ws_l = ws + n_o + n_s;
  a.ws_tab = (int32_t*)(ws + n_o + 2 * n_s);
  a.deterministic = (flags & AXL_DECODE_DETERMINISTIC) != 0 || deterministic_by_default();
  // Two workgroups fit a CU (LDS); the split kernel is persistent and strides over its work items.
  const dim3 grid(2 * cu_count());
  hipError_t err = hipSuccess;
  // With at most one block per workgroup (a bound the shapes give: the lengths live on the device) the
  // blocks are dealt by workgroup index and the counter is neither read nor zeroed.
  a.static_only = (int64_t)(a.B < kMaxBatch ? a.B : kMaxBatch) * a.Hv * a.nch <= (int64_t)grid.x;
  if (!(flags & AXL_DECODE_WORKSPACE_REUSED) && !a.static_only)
    hipLaunchKernelGGL(decode_plan_kernel, dim3(1), dim3(64), 0, stream, a.ticket);
#define AXL_DEC(E, DD, GG, NS, BB)                                                              \
  do {                                                                                          \
    using Tile = DecTile<DD, GG, NS>;                                                           \
    auto kern = decode_split_kernel<E, DD, GG, PAGED, NS, BB>;                                  \
    err = allow_dynamic_lds((const void*)kern, Tile::LDS_BYTES);                                \
    if (err == hipSuccess) {                                                                    \
      hipLaunchKernelGGL(kern, grid, dim3(256), Tile::LDS_BYTES, stream, s);                    \
      hipLaunchKernelGGL((decode_combine_kernel<E, DD, GG>), cgrid, dim3(256), 0, stream, s);   \
    }                                                                                           \
  } while (0)
  // The kernels keep per-sequence tables in LDS: larger batches go in slices of kMaxBatch (each
  // slice's combine kernel leaves the shared work counter at zero for the next slice).
  for (int b0 = 0; b0 < a.B && err == hipSuccess; b0 += kMaxBatch) {
    DecArgs s = a;
    s.B = a.B - b0 < kMaxBatch ? a.B - b0 : kMaxBatch;
    s.q = a.q + (size_t)b0 * a.Hq * a.d_real;
    s.out = a.out + (size_t)b0 * a.Hq * a.d_real;
    s.lengths = a.lengths + b0;
    if (PAGED) s.page_tables = a.page_tables + (size_t)b0 * a.pt_stride;
    else { s.k = a.k + b0 * a.ks.b; s.v = a.v + b0 * a.vs.b; }
    if (bias) s.bias = a.bias + b0 * a.bias_sb;
    s.ws_o = a.ws_o + (size_t)b0 * a.Hv * a.nch * gp * D;
    s.ws_m = a.ws_m + (size_t)b0 * a.Hv * a.nch * gp;
    s.ws_l = a.ws_l + (size_t)b0 * a.Hv * a.nch * gp;
    s.ws_tab = a.ws_tab + (size_t)b0 * a.Hv * a.nch;
    const dim3 cgrid(a.Hv, s.B);
    if (bias && D == 128) AXL_DEC(E, 128, 16, kStages128, true);
    else if (bias) AXL_DEC(E, 64, 16, kStages64, true);
    else if (D == 128 && gp == 4) AXL_DEC(E, 128, 4, kStages128, false);
    else if (D == 128 && gp == 8) AXL_DEC(E, 128, 8, kStages128, false);
    else if (D == 128) AXL_DEC(E, 128, 16, kStages128, false);
    else if (gp == 4) AXL_DEC(E, 64, 4, kStages64, false);
    else if (gp == 8) AXL_DEC(E, 64, 8, kStages64, false);
    else AXL_DEC(E, 64, 16, kStages64, false);
  }
#undef AXL_DEC
  if (err == hipSuccess) err = hipGetLastError();
  if (err != hipSuccess)
    return set_error(AXL_ERR_LAUNCH, "%s: launch failed: %s", who, hipGetErrorString(err));
  return AXL_OK;
}

template <bool PAGED>
static int launch_f32(DecArgs a, hipStream_t stream, const char* who) {
  const int D = width_of(a.d_real);
  const int gp = gp_of(a.G, a.bias != nullptr);
  a.ngrp = groups_of(a.G);
  a.Hv = a.Hkv * a.ngrp;
  a.chunk_pages = pick_chunk_pages(a.pps, (int64_t)a.B * a.Hv);
  if (a.chunk_pages > 256)
    return set_error(AXL_ERR_UNSUPPORTED, "%s: context longer than %d tokens", who, 256 * kMaxChunks * kPage);
  if (a.B > 65535) return set_error(AXL_ERR_UNSUPPORTED, "%s: more than 65535 sequences in fp32", who);
  a.nch = (a.pps + a.chunk_pages - 1) / a.chunk_pages;
  a.ticket = (int*)a.ws_o;
  a.ws_o += kWsHeaderFloats;
  float* ws = a.ws_o;
  const size_t n_o = (size_t)a.B * a.Hv * a.nch * gp * D;
  const size_t n_s = (size_t)a.B * a.Hv * a.nch * gp;
  a.ws_m = ws + n_o;
  a.ws_l = ws + n_o + n_s;
  a.ws_tab = (int32_t*)(ws + n_o + 2 * n_s);
  a.deterministic = 1;
  // One workgroup per live chunk writes that chunk's table entry; the work counter is not used (the
  // combine kernel still leaves it at zero).
  const dim3 grid(a.nch, a.Hv, a.B), cgrid(a.Hv, a.B);
#define AXL_DEC32(DD, GG)                                                                          \
  do {                                                                                              \
    hipLaunchKernelGGL((decode_split_f32_kernel<DD, GG, PAGED>), grid, dim3(256), 0, stream, a);    \
    hipLaunchKernelGGL((decode_combine_kernel<ElemF32, DD, GG>), cgrid, dim3(256), 0, stream, a);   \
  } while (0)
  if (D == 128 && gp == 4) AXL_DEC32(128, 4);
  else if (D == 128 && gp == 8) AXL_DEC32(128, 8);
  else if (D == 128) AXL_DEC32(128, 16);
  else if (gp == 4) AXL_DEC32(64, 4);
  else if (gp == 8) AXL_DEC32(64, 8);
  else AXL_DEC32(64, 16);
#undef AXL_DEC32
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return set_error(AXL_ERR_LAUNCH, "%s: launch failed: %s", who, hipGetErrorString(err));
  return AXL_OK;
}

int launch_paged_decode(const AxlPagedDecodeParams& p, hipStream_t stream) {
  DecArgs a{};
  a.q = (const __bf16*)p.q; a.k = (const __bf16*)p.k_pages; a.v = (const __bf16*)p.v_pages;
  a.page_tables = p.page_tables; a.lengths = p.lengths; a.out = (__bf16*)p.out;
  a.ws_o = (float*)p.workspace;
  a.B = p.batch; a.Hq = p.num_q_heads; a.Hkv = p.num_kv_heads; a.G = p.num_q_heads / p.num_kv_heads;
  a.page_shift = page_shift_of(p.page_size);   // the entry point has checked the page size
  a.pt_stride = p.pages_per_seq;
  a.num_pages = p.num_pages; a.pps = p.pages_per_seq << a.page_shift; a.kv_len = p.pages_per_seq * p.page_size;
  a.d_real = p.head_dim;
  a.window = p.sliding_window < 0 ? -1 : p.sliding_window;
  a.scale = p.softmax_scale;
  set_bias(a, p.bias, p.softmax_scale);
  if (p.dtype == AXL_F32) return launch_f32<true>(a, stream, "axl_paged_decode");
  return p.dtype == AXL_F16 ? launch_common<ElemF16, true>(a, p.flags, stream, "axl_paged_decode")
                            : launch_common<ElemBf16, true>(a, p.flags, stream, "axl_paged_decode");
}

// ---------------------------------------------------------------------------------------------
// Allocation-free variant of the paged decode: the split-K workspace (partial records, record table,
// work counter) is this file-scope device array instead of caller memory.  Every GPU the library runs
// on holds its own copy until the process ends; `scratch` itself is a host-side stand-in, the device
// address comes from hipGetSymbolAddress, once per device.
// ---------------------------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = AXL_PAGED_DECODE_STATIC_MAX_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, once resolved

// Device address of this device's copy of `scratch` (the current device is the one the call runs on).
static int static_scratch(void** ptr, const char* who) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return set_error(AXL_ERR_LAUNCH, "%s: hipGetDevice: %s", who, hipGetErrorString(err));
  if (dev < 0 || dev >= kMaxDevices) return set_error(AXL_ERR_UNSUPPORTED, "%s: device index %d", who, dev);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !p)
      return set_error(AXL_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch): %s", who, hipGetErrorString(err));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return AXL_OK;
}

int launch_paged_decode_static(const AxlPagedDecodeParams& p, hipStream_t stream) {
  const char* who = "axl_paged_decode_static";
  const size_t need = paged_decode_workspace_bytes(p);
  if (need > kStaticScratchBytes)
    return set_error(AXL_ERR_WORKSPACE,
                     "%s: these shapes need %zu bytes of split-K scratch, the built-in buffer holds %zu "
                     "(use axl_paged_decode with a caller workspace)", who, need, kStaticScratchBytes);
  void* ws = nullptr;
  const int rc = static_scratch(&ws, who);
  if (rc != AXL_OK) return rc;
  AxlPagedDecodeParams q = p;
  q.workspace = ws;  // the resolved device address, never the array's name
  q.workspace_bytes = kStaticScratchBytes;
  // The buffer keeps the previous call's contents (possibly of other shapes, possibly of a call that
  // was captured and never replayed): the work counter is zeroed by a kernel on every call.
  q.flags &= ~AXL_DECODE_WORKSPACE_REUSED;
  return launch_paged_decode(q, stream);
}

int launch_decode(const AxlDecodeParams& p, hipStream_t stream) {
  DecArgs a{};
  a.q = (const __bf16*)p.q; a.k = (const __bf16*)p.k; a.v = (const __bf16*)p.v;
  a.page_tables = nullptr; a.lengths = p.lengths; a.out = (__bf16*)p.out;
  a.ws_o = (float*)p.workspace;
  a.ks = Strides3{p.k_strides.batch, p.k_strides.seq, p.k_strides.head};
  a.vs = Strides3{p.v_strides.batch, p.v_strides.seq, p.v_strides.head};
  a.B = p.batch; a.Hq = p.num_q_heads; a.Hkv = p.num_kv_heads; a.G = p.num_q_heads / p.num_kv_heads;
  a.num_pages = 0; a.pps = (p.kv_len + kPage - 1) / kPage; a.kv_len = p.kv_len;
  a.page_shift = 0; a.pt_stride = 0;
  a.d_real = p.head_dim;
  a.window = p.sliding_window < 0 ? -1 : p.sliding_window;
  a.scale = p.softmax_scale;
  set_bias(a, p.bias, p.softmax_scale);
  if (p.dtype == AXL_F32) return launch_f32<false>(a, stream, "axl_decode");
  return p.dtype == AXL_F16 ? launch_common<ElemF16, false>(a, p.flags, stream, "axl_decode")
                            : launch_common<ElemBf16, false>(a, p.flags, stream, "axl_decode");
}

}  // namespace axl
