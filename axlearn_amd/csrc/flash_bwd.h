// Argument block shared by the backward kernels (delta pre-pass, dK/dV, dQ).
#pragma once

#include "common.h"

namespace axl {

struct BwdArgs {
  const void* q;
  const void* k;
  const void* v;
  const void* out;
  const void* dout;
  const float* lse;
  float* ndelta; // workspace [B, Hq, T]: -rowsum(out * dO); negated so that a dP accumulator chain can start from it
  float* lse2;   // workspace [B, Hq, T]: -lse * log2(e), the exponent offset of the dK/dV kernel
  void* ds;      // workspace: dS blocks left by the dK/dV kernel for the streaming dQ kernel (spill path), or nullptr
  void* dq;
  void* dk;
  void* dv;
  const int32_t* seg;
  const int2* seg_tbl;  // workspace [B, T / 32]: smallest and largest segment id of every 32 rows (with seg)
  int2* kb_tbl;         // workspace [B, S / 128]: the query tiles [first, end) whose dS each key block's dK/dV
                        // workgroups store (spill path under a sliding window or segment ids), or nullptr
  Strides3 qs, ks, vs, os, dos, dqs, dks, dvs;
  int B, T, S, Hq, Hkv;
  int stat_hq;  // query heads of the [B, heads, T] statistics (ndelta, lse2): Hq, or more when the
                // launch covers a slice of the heads and the pointers start at the slice's first head
  int mask_kind, window, q_off;
  float scale;
  int d_real;   // head_dim of the tensors: a multiple of 8, at most the compiled width (16-bit kernels without
                // bias / dropout mask).  Operand fragments are zero past it, tile loads fetch slice 0 of the row in
                // place of the slices past it (finite values that only ever meet those zeros or end up in
                // output columns that are not stored), stores leave the columns past it out.
  int kb_per_wg;  // key blocks (of 128 keys) a dK/dV workgroup works through: 1, or 2 (a block and its mirror image)
  AuxArgs aux;  // dense bias / dropout mask (read only by the AUX instantiations)
};

// Most key blocks (of 128 keys) the spill path handles when the stored tiles depend on the key block.
constexpr int kMaxKbRanged = 512;

// dS workspace of the spill path (causal or sliding-window mask, q_pos_offset 0, q_len == kv_len).  A block is the dS
// of 32 queries x 32 keys as [query half 2][key 32][16 queries] in the input dtype: 2 KB.  Query tile
// t = 4a + r (32 rows) of a head has a run of ds_run_blocks(t) = 4(a+1) blocks, one per 32 keys that the
// 128 query rows of block a can see.  Per (batch, kv head) pair the runs are ordered by tile, then by
// query head of the group: the workgroups of a pair's dK/dV launch, which walk the tiles in step and
// loop over the group's heads, then write next to each other, and a query tile's run stays contiguous
// for the dQ kernel.
constexpr int kDsBlockBytes = 2048;
__host__ __device__ inline int64_t ds_blocks_per_head(int T) {
  const int64_t A = T / 128;
  return 8 * A * (A + 1);
}
__host__ __device__ inline int64_t ds_run_blocks(int t) { return 4 * (int64_t)((t >> 2) + 1); }
__host__ __device__ inline int64_t ds_tile_offset(int t) {  // blocks of one head ahead of query tile t
  const int64_t a = t >> 2, r = t & 3;
  return 4 * (2 * a + r) * (a + 1);
}
// First block of the run of (pair, query tile t, head hh of the group of G), in blocks.
__host__ __device__ inline int64_t ds_run_start(int64_t pair, int T, int G, int t, int hh) {
  return G * (pair * ds_blocks_per_head(T) + ds_tile_offset(t)) + hh * ds_run_blocks(t);
}

// Enqueues the dK/dV kernel for `dtype` AXL_BF16 or AXL_F16 and head_dim 64 or 128; `aux` selects
// the instantiation that reads the dense bias / dropout mask.  With a.ds set (and no bias / dropout
// mask, causal or sliding-window mask, q_off 0, T == S) the kernel also stores dS for
// launch_bwd_dq_stream, and with a.kb_tbl set the range of query tiles each key block stored.
hipError_t launch_bwd_dkdv(const BwdArgs& a, int dtype, int head_dim, bool aux, hipStream_t stream);

// Enqueues the streaming dQ kernel, dq = scale * dS k from the dS blocks in a.ds (with a.kb_tbl set:
// from the blocks that table says were stored).
hipError_t launch_bwd_dq_stream(const BwdArgs& a, int dtype, int head_dim, hipStream_t stream);

// Enqueues the dQ kernel (no dense bias / dropout mask) for `dtype` AXL_BF16 or AXL_F16 and head_dim
// 64 or 128.  With `fuse_delta` it also writes delta and the scaled lse into the workspace (instead
// of reading them), for a dK/dV kernel enqueued after it.
hipError_t launch_bwd_dq(const BwdArgs& a, int dtype, int head_dim, bool fuse_delta, hipStream_t stream);

// Enqueues the fp32 dK/dV and / or dQ kernels (`phases`: AXL_BWD_DKDV, AXL_BWD_DQ) for head_dim 64
// or 128; they read delta from the workspace and honour the dense bias / dropout mask.
hipError_t launch_bwd_f32(const BwdArgs& a, int head_dim, int phases, hipStream_t stream);

}  // namespace axl
