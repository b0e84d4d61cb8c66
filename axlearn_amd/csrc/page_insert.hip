// Insertion of one new token per sequence into a paged KV pool, in place.
//
// Replaces axlearn/common/kv_cache/paged_kv_cache_gpu_kernel.py:16-60 (`_scatter_pages_kernel` and
// its launcher), as called from `PagedKVCache.extend_step`
// (axlearn/common/kv_cache/paged_kv_cache.py:213-240).  Pure addressing and byte copies:
//   pos = key_positions[b]; live iff 0 <= pos < page_size * pages_per_seq           (:26)
//   page = page_indices[b][pos / page_size]; offset = pos % page_size               (:28-29)
//   pages[h][page][offset][:] = proj[b][h][:]  iff live and page != 0               (:31-33)
// Page 0 is the padding page and is never written (paged_kv_cache.py:120).  A page index outside
// the pool is dropped, as the reference's scatter does with mode="drop" (paged_kv_cache.py:56-58).
#include "common.h"

namespace axl {

struct InsertArgs {
  char* k_pages;            // [Hkv, P, page_size, D], may be null
  char* v_pages;            // same, may be null
  const char* k_proj;       // [B, Hkv, D] through strides (bytes)
  const char* v_proj;
  const int32_t* page_indices;   // [B, pps]
  const int32_t* key_positions;  // [B] or a single value broadcast over the batch
  int64_t kp_b, kp_h, vp_b, vp_h;  // proj strides in bytes
  int B, Hkv, num_pages, page_size, pps;
  int row_bytes;            // D * element size
  int pos_stride;           // 0 (broadcast) or 1
};

__global__ __launch_bounds__(256) void page_insert_kernel(const InsertArgs a) {
  const int b = blockIdx.x;
  const int pos = a.key_positions[(int64_t)b * a.pos_stride];
  if (pos < 0 || pos >= a.page_size * a.pps) return;
  const int page = a.page_indices[(int64_t)b * a.pps + pos / a.page_size];
  if (page <= 0 || page >= a.num_pages) return;
  const int offset = pos % a.page_size;
  const int chunks = a.row_bytes / 16;  // 16-byte pieces per row
  for (int i = threadIdx.x; i < a.Hkv * chunks; i += blockDim.x) {
    const int h = i / chunks, c = i % chunks;
    const int64_t dst = (((int64_t)h * a.num_pages + page) * a.page_size + offset) * a.row_bytes + 16 * c;
    if (a.k_pages) *(uint4*)(a.k_pages + dst) = *(const uint4*)(a.k_proj + b * a.kp_b + h * a.kp_h + 16 * c);
    if (a.v_pages) *(uint4*)(a.v_pages + dst) = *(const uint4*)(a.v_proj + b * a.vp_b + h * a.vp_h + 16 * c);
  }
}

int launch_page_insert(const AxlPageInsertParams& p, hipStream_t stream) {
  const int es = p.dtype == AXL_F32 ? 4 : 2;
  InsertArgs a{};
  a.k_pages = (char*)p.k_pages; a.v_pages = (char*)p.v_pages;
  a.k_proj = (const char*)p.k_proj; a.v_proj = (const char*)p.v_proj;
  a.page_indices = p.page_indices; a.key_positions = p.key_positions;
  a.kp_b = p.k_proj_batch_stride * es; a.kp_h = p.k_proj_head_stride * es;
  a.vp_b = p.v_proj_batch_stride * es; a.vp_h = p.v_proj_head_stride * es;
  a.B = p.batch; a.Hkv = p.num_kv_heads; a.num_pages = p.num_pages; a.page_size = p.page_size;
  a.pps = p.pages_per_seq; a.row_bytes = p.head_dim * es;
  a.pos_stride = p.broadcast_positions ? 0 : 1;
  hipLaunchKernelGGL(page_insert_kernel, dim3(p.batch), dim3(256), 0, stream, a);
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess)
    return set_error(AXL_ERR_LAUNCH, "axl_paged_kv_insert: launch failed: %s", hipGetErrorString(err));
  return AXL_OK;
}

}  // namespace axl
