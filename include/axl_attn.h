/*
 * axl_attn.h -- C ABI of libaxl_attn_hip.so: hand-written CDNA4 (gfx950) attention kernels that
 * stand behind AXLearn's `flash_attention_implementation` dispatch.
 *
 * Conventions shared by every entry point:
 *   - plain C types only; every pointer is a DEVICE pointer owned by the caller (inputs, outputs and
 *     workspace).  The library never allocates, frees or synchronises: each call only enqueues
 *     kernels on `stream` (a hipStream_t passed as void*; NULL = the default stream).
 *   - returns 0 on success or a negative AxlStatus; the message for the calling thread's last
 *     failure is available from axl_last_error().  No C++ exception crosses the boundary.
 *   - tensors are dense in their last dimension; the other strides are given in ELEMENTS.
 *   - masking follows axlearn/common/attention_bias.py: a query at position qp may attend a key at
 *     position kp iff   causal: qp >= kp   (:652-658);   sliding window w: qp >= kp && qp - kp <= w,
 *     i.e. w+1 keys (:771-790);   segment ids: seg[q] == seg[k], id 0 included (:876-882).
 *     Query position of row t is t + q_pos_offset; key position of row s is s.
 *   - GQA: query head n reads kv head n / (num_q_heads / num_kv_heads)
 *     (axlearn/common/attention.py:2344).
 */
#ifndef AXL_ATTN_H_
#define AXL_ATTN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AXL_ATTN_ABI_VERSION 2

typedef enum AxlStatus {
  AXL_OK = 0,
  AXL_ERR_INVALID_ARGUMENT = -1, /* shapes / pointers that make no sense                      */
  AXL_ERR_UNSUPPORTED = -2,      /* legal request this library has no kernel for               */
  AXL_ERR_WORKSPACE = -3,        /* workspace missing or too small                             */
  AXL_ERR_LAUNCH = -4            /* hipLaunchKernel reported an error                          */
} AxlStatus;

typedef enum AxlDtype { AXL_BF16 = 0, AXL_F32 = 1 } AxlDtype;

typedef enum AxlMaskKind {
  AXL_MASK_NONE = 0,
  AXL_MASK_CAUSAL = 1,
  AXL_MASK_SLIDING_WINDOW = 2 /* causal + window; see above */
} AxlMaskKind;

/* [batch, seq, heads, head_dim] tensor: strides for batch, seq and heads in elements. */
typedef struct AxlStrides {
  int64_t batch;
  int64_t seq;
  int64_t head;
} AxlStrides;

/*
 * Flash-attention forward.
 * Replaces: `flash_attention` / `_flash_attention_impl` -> pallas_call(mha_forward)
 *   (axlearn/common/flash_attention/gpu_attention.py:250-287, 293-425) as reached from
 *   `PallasGPUFlashAttention.__call__` (:964-992), without materialising repeated KV heads.
 *   q [B,T,Hq,D]; k,v [B,S,Hkv,D]; out [B,T,Hq,D] (dtype of q); lse [B,Hq,T] fp32 = natural-log
 *   sum-exp of the scaled, masked logits (the residual the backward needs, :241); lse may be NULL.
 *   segment_ids [B,T] int32 or NULL (needs T == S).
 * Supported: dtype bf16 or f32; head_dim 64 or 128; T % 128 == 0 and S % 128 == 0.
 */
typedef struct AxlFlashFwdParams {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse;
  const int32_t* segment_ids;
  AxlStrides q_strides, k_strides, v_strides, out_strides;
  int32_t batch, q_len, kv_len, num_q_heads, num_kv_heads, head_dim;
  int32_t dtype;          /* AxlDtype of q, k, v, out */
  int32_t mask_kind;      /* AxlMaskKind */
  int32_t sliding_window; /* left context w (keeps w+1 keys); used when mask_kind == SLIDING */
  int32_t q_pos_offset;   /* position of query row 0 */
  float softmax_scale;    /* > 0; multiplies q.k before masking and softmax */
  const float* logit_sink; /* [Hq] fp32 or NULL: one extra logit per row of head h that takes part in
                              the softmax (and in lse) but has no value row, so the attention
                              weights of the real keys sum to less than 1
                              (axlearn/common/attention.py:608-626; not scaled, never masked) */
} AxlFlashFwdParams;

int axl_flash_fwd(const AxlFlashFwdParams* params, void* stream);

/*
 * Flash-attention backward.
 * Replaces: `_mha_backward` (delta pre-pass, pallas_call(_mha_backward_kernel_dkdv) and
 *   pallas_call(_mha_backward_kernel_dq); axlearn/common/flash_attention/gpu_attention.py:621-786).
 *   Inputs are the forward's residuals (q, k, v, out, lse) and d_out; outputs dq [B,T,Hq,D],
 *   dk, dv [B,S,Hkv,D] in the dtype of q/k/v.  dk/dv are already summed over the Hq/Hkv query
 *   heads of each kv head (what autodiff of `repeat_kv_heads` does in the reference).
 *   workspace: axl_flash_bwd_workspace_bytes(params) bytes of device scratch (holds delta).
 *   With a logit sink, dq/dk/dv need nothing beyond an lse that includes the sink; its own gradient
 *   is a per-head reduction of delta (the Pallas kernels have no sink: gpu_attention.py:957-959
 *   declines it, so this follows the XLA path, flash_attention/common.py:502-511).
 */
typedef struct AxlFlashBwdParams {
  const void* q;
  const void* k;
  const void* v;
  const void* out;
  const void* d_out;
  const float* lse;
  void* dq;
  void* dk;
  void* dv;
  const int32_t* segment_ids;
  AxlStrides q_strides, k_strides, v_strides, out_strides, d_out_strides;
  AxlStrides dq_strides, dk_strides, dv_strides;
  int32_t batch, q_len, kv_len, num_q_heads, num_kv_heads, head_dim;
  int32_t dtype;
  int32_t mask_kind;
  int32_t sliding_window;
  int32_t q_pos_offset;
  float softmax_scale;
  void* workspace;
  size_t workspace_bytes;
  const float* logit_sink; /* [Hq] fp32 or NULL; must be what the forward that produced lse was given */
  float* d_logit_sink;     /* [Hq] fp32 out or NULL: -sum over (b, t) of exp(sink - lse) * delta,
                              written (not accumulated) by the DELTA phase */
} AxlFlashBwdParams;

size_t axl_flash_bwd_workspace_bytes(const AxlFlashBwdParams* params);
int axl_flash_bwd(const AxlFlashBwdParams* params, void* stream);

/*
 * Runs a subset of the backward's kernels, for per-kernel timing and profiling: `phases` is a
 * bit mask of AXL_BWD_DELTA (delta pre-pass, gpu_attention.py:653-658), AXL_BWD_DKDV
 * (`_mha_backward_kernel_dkdv`, :436-528) and AXL_BWD_DQ (`_mha_backward_kernel_dq`, :533-616), the
 * three launches `_mha_backward` makes.  The dK/dV and dQ phases read the delta a previous DELTA
 * phase left in the same workspace.  axl_flash_bwd(p, s) == axl_flash_bwd_phases(p, 7, s).
 */
#define AXL_BWD_DELTA 1
#define AXL_BWD_DKDV 2
#define AXL_BWD_DQ 4
int axl_flash_bwd_phases(const AxlFlashBwdParams* params, int phases, void* stream);

/*
 * Paged-attention decode (one query token per sequence).
 * Replaces: `GPUPagedAttention.__call__` -> vmap(_paged_attention_unbatched) ->
 *   pallas_call(paged_attention_*) + the XLA combine
 *   (axlearn/common/flash_attention/gpu_paged_attention.py:325-379, 164-296, 38-152).
 *   q [B,Hq,D]; k_pages, v_pages [Hkv, num_pages, page_size, D]; page_tables [B, pages_per_seq]
 *   int32: token j of sequence b is k_pages[h][page_tables[b][j / page_size]][j % page_size]
 *   (axlearn/common/kv_cache/paged_kv_cache.py:21-34); lengths [B] int32: keys j >= lengths[b] are
 *   masked (:100); the query sits at position lengths[b]-1 (:344).  As in `reconstruct_kv`, a page
 *   index in [-num_pages, 0) counts from the end of the pool and any other index outside
 *   [0, num_pages) reads as zeros.  out [B,Hq,D] in the dtype of q.
 *   sliding_window < 0 disables the window; otherwise keys with (len-1) - j > w are masked too.
 *   workspace: axl_paged_decode_workspace_bytes(params) bytes (fp32 split-K partial records, a
 *   record table and two work counters; its contents need not be initialised or preserved).
 *   Up to 16 query heads per kv head; head_dim 64 or 128; page_size 16; bf16.
 *   Work is handed to workgroups by timing, so two calls on the same inputs may group the fp32
 *   partial sums differently (differences far below bf16 resolution before the final rounding).
 *   With AXL_DECODE_DETERMINISTIC=1 in the environment the decomposition is fixed and the result
 *   is reproducible bit for bit, at a few percent of bandwidth.  The same holds for axl_decode.
 */
typedef struct AxlPagedDecodeParams {
  const void* q;
  const void* k_pages;
  const void* v_pages;
  const int32_t* page_tables;
  const int32_t* lengths;
  void* out;
  int32_t batch, num_q_heads, num_kv_heads, head_dim;
  int32_t num_pages, page_size, pages_per_seq;
  int32_t dtype;
  int32_t sliding_window;
  float softmax_scale;
  void* workspace;
  size_t workspace_bytes;
} AxlPagedDecodeParams;

size_t axl_paged_decode_workspace_bytes(const AxlPagedDecodeParams* params);
int axl_paged_decode(const AxlPagedDecodeParams* params, void* stream);

/*
 * Flash-decoding over a contiguous KV cache (one query token per sequence).
 * Replaces: `GPUDecoding.__call__` -> vmap(_decode_attn_unbatched) ->
 *   pallas_call(flash_decoding_forward) + the XLA combine
 *   (axlearn/common/flash_attention/gpu_decoding.py:304-352, 192-283, 71-173).
 *   q [B,Hq,D]; k, v [B,S,Hkv,D] with strides; lengths [B] int32 (= target_positions[:, -1] + 1,
 *   :314); out [B,Hq,D].
 */
typedef struct AxlDecodeParams {
  const void* q;
  const void* k;
  const void* v;
  const int32_t* lengths;
  void* out;
  AxlStrides k_strides, v_strides;
  int32_t batch, kv_len, num_q_heads, num_kv_heads, head_dim;
  int32_t dtype;
  int32_t sliding_window;
  float softmax_scale;
  void* workspace;
  size_t workspace_bytes;
} AxlDecodeParams;

size_t axl_decode_workspace_bytes(const AxlDecodeParams* params);
int axl_decode(const AxlDecodeParams* params, void* stream);

/*
 * Insertion of one new token per sequence into the paged KV pools, in place.
 * Replaces: `gpu_scatter_update_pages_shmap_fn` / `_scatter_pages_kernel`
 *   (axlearn/common/kv_cache/paged_kv_cache_gpu_kernel.py:16-60) as called for K and for V from
 *   `PagedKVCache.extend_step` (axlearn/common/kv_cache/paged_kv_cache.py:213-240); both pools are
 *   updated by one call (either pool/proj pair may be NULL).
 *   k_pages, v_pages [Hkv, num_pages, page_size, D]; k_proj, v_proj: the new token's projections,
 *   element (b, h, :) at  b * batch_stride + h * head_stride  (elements), which covers both the
 *   layer's [B,1,Hkv,D] and the kernel's [Hkv,B,1,D] layouts; page_indices [B, pages_per_seq] int32;
 *   key_positions [B] int32 (or one value for all sequences when broadcast_positions != 0).
 *   For sequence b with pos = key_positions[b]: nothing is written unless
 *   0 <= pos < page_size * pages_per_seq (:26); page = page_indices[b][pos / page_size]; the row
 *   pages[h][page][pos % page_size][:] is overwritten for every h unless page == 0, the padding page
 *   (:31, paged_kv_cache.py:120), or page lies outside the pool (dropped, paged_kv_cache.py:56-58).
 *   Sequences must not share a live page (as in the reference: unique_indices).
 */
typedef struct AxlPageInsertParams {
  void* k_pages;
  void* v_pages;
  const void* k_proj;
  const void* v_proj;
  const int32_t* page_indices;
  const int32_t* key_positions;
  int64_t k_proj_batch_stride, k_proj_head_stride;
  int64_t v_proj_batch_stride, v_proj_head_stride;
  int32_t batch, num_kv_heads, head_dim;
  int32_t num_pages, page_size, pages_per_seq;
  int32_t dtype;               /* AxlDtype of the pools and projections */
  int32_t broadcast_positions; /* key_positions holds a single value */
} AxlPageInsertParams;

int axl_paged_kv_insert(const AxlPageInsertParams* params, void* stream);

/* Message describing the calling thread's most recent failure ("" if none). Never NULL. */
const char* axl_last_error(void);

/* AXL_ATTN_ABI_VERSION the library was built with. */
int axl_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* AXL_ATTN_H_ */
