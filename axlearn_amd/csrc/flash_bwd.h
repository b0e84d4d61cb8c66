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
  void* dq;
  void* dk;
  void* dv;
  const int32_t* seg;
  Strides3 qs, ks, vs, os, dos, dqs, dks, dvs;
  int B, T, S, Hq, Hkv;
  int mask_kind, window, q_off;
  float scale;
  AuxArgs aux;  // dense bias / dropout mask (read only by the AUX instantiations)
};

// Enqueues the dK/dV kernel for `dtype` AXL_BF16 or AXL_F16 and head_dim 64 or 128; `aux` selects
// the instantiation that reads the dense bias / dropout mask.
hipError_t launch_bwd_dkdv(const BwdArgs& a, int dtype, int head_dim, bool aux, hipStream_t stream);

// Enqueues the dQ kernel (no dense bias / dropout mask) for `dtype` AXL_BF16 or AXL_F16 and head_dim
// 64 or 128.  With `fuse_delta` it also writes delta and the scaled lse into the workspace (instead
// of reading them), for a dK/dV kernel enqueued after it.
hipError_t launch_bwd_dq(const BwdArgs& a, int dtype, int head_dim, bool fuse_delta, hipStream_t stream);

// Enqueues the fp32 dK/dV and / or dQ kernels (`phases`: AXL_BWD_DKDV, AXL_BWD_DQ) for head_dim 64
// or 128; they read delta from the workspace and honour the dense bias / dropout mask.
hipError_t launch_bwd_f32(const BwdArgs& a, int head_dim, int phases, hipStream_t stream);

}  // namespace axl
