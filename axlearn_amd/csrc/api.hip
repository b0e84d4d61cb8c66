// extern "C" entry points of libaxl_attn_hip.so: argument validation, error reporting, dispatch to
// the kernel launchers.  Nothing here allocates device memory or synchronises.
#include <cstdarg>
#include <cstdio>
#include <cmath>
#include <initializer_list>
#include <mutex>
#include <unordered_map>

#include "common.h"

namespace axl {

static thread_local char g_last_error[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int launch_flash_fwd(const AxlFlashFwdParams& p, hipStream_t stream);
int launch_flash_bwd(const AxlFlashBwdParams& p, int phases, hipStream_t stream);
size_t flash_bwd_workspace_bytes(const AxlFlashBwdParams& p);
int launch_paged_decode(const AxlPagedDecodeParams& p, hipStream_t stream);
size_t paged_decode_workspace_bytes(const AxlPagedDecodeParams& p);
int launch_paged_decode_static(const AxlPagedDecodeParams& p, hipStream_t stream);
int launch_decode(const AxlDecodeParams& p, hipStream_t stream);
size_t decode_workspace_bytes(const AxlDecodeParams& p);
int launch_page_insert(const AxlPageInsertParams& p, hipStream_t stream);

// Compute units of the current device (256 on an MI355X; that figure too if the query fails), looked up once.
int cu_count() {
  static int n = 0;
  if (n == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      n = v;
    else
      n = 256;
  }
  return n;
}

hipError_t allow_dynamic_lds(const void* kernel, int bytes) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  const uint64_t key = (uint64_t)reinterpret_cast<uintptr_t>(kernel) ^ ((uint64_t)(dev + 1) << 56);
  // The pair this thread set (or found set) last: repeated launches of one kernel take no lock.
  static thread_local uint64_t last_key = 0;
  static thread_local int last_bytes = 0;
  if (last_key == key && last_bytes >= bytes) return hipSuccess;
  static std::mutex mu;
  static std::unordered_map<uint64_t, int> granted;  // (kernel, device) -> limit already set
  std::lock_guard<std::mutex> lock(mu);
  auto it = granted.find(key);
  if (it == granted.end() || it->second < bytes) {
    err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (err != hipSuccess) return err;
    granted[key] = bytes;
  }
  last_key = key;
  last_bytes = bytes;
  return hipSuccess;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

static bool strides_ok(const AxlStrides& s, int elem_bytes) {
  // 16-byte vector loads along head_dim need every row start 16-byte aligned.
  const int64_t m = 16 / elem_bytes;
  return s.batch % m == 0 && s.seq % m == 0 && s.head % m == 0;
}

// Shape rules shared by forward and backward; mirrors BaseFlashAttention.is_supported
// (axlearn/common/flash_attention/common.py:232-275) for the "makes no sense" cases and
// PallasGPUFlashAttention.is_supported (gpu_attention.py:939-961) for the unsupported ones.
static int check_flash_shapes(const char* who, int batch, int q_len, int kv_len, int hq, int hkv,
                              int d, int dtype, int mask_kind, int window, float scale,
                              const int32_t* seg) {
  if (batch <= 0 || q_len <= 0 || kv_len <= 0 || hq <= 0 || hkv <= 0 || d <= 0)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: non-positive dimension", who);
  if (hq % hkv != 0)
    return set_error(AXL_ERR_INVALID_ARGUMENT,
                     "%s: num_q_heads %d is not divisible by num_kv_heads %d", who, hq, hkv);
  if (!(scale > 0.f) || !std::isfinite(scale))
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: softmax_scale must be finite and > 0", who);
  if (dtype != AXL_BF16 && dtype != AXL_F32 && dtype != AXL_F16)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: unknown dtype %d", who, dtype);
  if (mask_kind < AXL_MASK_NONE || mask_kind > AXL_MASK_SLIDING_WINDOW)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: unknown mask_kind %d", who, mask_kind);
  if (mask_kind == AXL_MASK_SLIDING_WINDOW && window < 0)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: sliding_window must be >= 0", who);
  if (seg && q_len != kv_len)
    return set_error(AXL_ERR_INVALID_ARGUMENT,
                     "%s: segment_ids need q_len == kv_len (got %d vs %d)", who, q_len, kv_len);
  if (dtype == AXL_F32 ? (d != 64 && d != 128) : (d > 128 || d % 8 != 0))
    return set_error(AXL_ERR_UNSUPPORTED, "%s: head_dim %d (supported: 64 and 128; in bf16 / f16 any multiple of 8 up to 128)",
                     who, d);
  if (q_len % 128 != 0 || kv_len % 128 != 0)
    return set_error(AXL_ERR_UNSUPPORTED, "%s: q_len %d / kv_len %d not divisible by 128", who,
                     q_len, kv_len);
  return AXL_OK;
}

// A head_dim between the compiled widths (16-bit kernels): the kernels run at the next width on the
// tensors as they are.  Their tile loads address a second 1 KB group of rows relative to the first,
// which needs rows at least as far apart as the compiled width, and the bias / dropout instantiations
// have no such form.
static int check_odd_head_dim(const char* who, int d, bool aux, std::initializer_list<const AxlStrides*> tensors) {
  if (d == 64 || d == 128) return AXL_OK;
  if (aux)
    return set_error(AXL_ERR_UNSUPPORTED, "%s: head_dim %d with a bias or dropout mask (supported: 64, 128)", who, d);
  const int width = d <= 64 ? 64 : 128;
  for (const AxlStrides* s : tensors)
    if (s->seq < width)
      return set_error(AXL_ERR_UNSUPPORTED, "%s: head_dim %d needs rows at least %d elements apart", who, d, width);
  return AXL_OK;
}

AuxArgs make_aux_args(const AxlAttnAux& x, float softmax_scale) {
  AuxArgs a;
  const int es = x.bias_dtype == AXL_F32 ? 4 : 2;
  a.bias = (const char*)x.bias;
  a.drop = x.dropout_mask;
  a.bias_sb = x.bias_batch_stride * es; a.bias_sh = x.bias_head_stride * es; a.bias_sr = x.bias_row_stride * es;
  a.drop_sb = x.drop_batch_stride; a.drop_sh = x.drop_head_stride; a.drop_sr = x.drop_row_stride;
  a.bias_f32 = x.bias_dtype == AXL_F32;
  a.inv_scale = 1.0f / softmax_scale;
  a.keep_scale = x.dropout_mask ? 1.0f / (1.0f - x.dropout_rate) : 1.0f;
  return a;
}

// The kernels read 8 consecutive bias elements / mask bytes per access (4 in the fp32 forward).
int check_aux(const char* who, const AxlAttnAux& x, int batch, int hq, int q_len, int kv_len) {
  (void)batch; (void)hq; (void)q_len;
  if (x.bias) {
    if (x.bias_dtype == AXL_F16)
      return set_error(AXL_ERR_UNSUPPORTED, "%s: an fp16 bias is not supported (pass it as fp32 or bf16)", who);
    if (x.bias_dtype != AXL_BF16 && x.bias_dtype != AXL_F32)
      return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: unknown bias dtype %d", who, x.bias_dtype);
    const int64_t m = x.bias_dtype == AXL_F32 ? 4 : 8;
    if (x.bias_batch_stride < 0 || x.bias_head_stride < 0 || x.bias_row_stride < kv_len)
      return set_error(AXL_ERR_INVALID_ARGUMENT,
                       "%s: bias strides must be >= 0 and its row stride >= kv_len", who);
    if (!aligned16(x.bias) || x.bias_batch_stride % m || x.bias_head_stride % m || x.bias_row_stride % m)
      return set_error(AXL_ERR_UNSUPPORTED, "%s: bias rows must be 16-byte aligned", who);
  }
  if (x.dropout_mask) {
    if (!(x.dropout_rate >= 0.f) || !(x.dropout_rate < 1.f))
      return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: dropout_rate must be in [0, 1)", who);
    if (x.drop_batch_stride < 0 || x.drop_head_stride < 0 || x.drop_row_stride < kv_len)
      return set_error(AXL_ERR_INVALID_ARGUMENT,
                       "%s: dropout mask strides must be >= 0 and its row stride >= kv_len", who);
    if ((reinterpret_cast<uintptr_t>(x.dropout_mask) & 7) || x.drop_batch_stride % 8 ||
        x.drop_head_stride % 8 || x.drop_row_stride % 8)
      return set_error(AXL_ERR_UNSUPPORTED, "%s: dropout mask rows must be 8-byte aligned", who);
  } else if (x.dropout_rate != 0.f) {
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: dropout_rate without a dropout_mask", who);
  }
  return AXL_OK;
}

}  // namespace axl

using namespace axl;

extern "C" {

int axl_paged_kv_insert(const AxlPageInsertParams* p, void* stream) {
  using namespace axl;
  const char* who = "axl_paged_kv_insert";
  if (!p) return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: null params", who);
  if (p->batch <= 0 || p->num_kv_heads <= 0 || p->head_dim <= 0 || p->num_pages <= 0 ||
      p->page_size <= 0 || p->pages_per_seq <= 0)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: non-positive dimension", who);
  if (p->dtype != AXL_BF16 && p->dtype != AXL_F32 && p->dtype != AXL_F16)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: unknown dtype %d", who, p->dtype);
  if (!p->page_indices || !p->key_positions)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: null page_indices / key_positions", who);
  if ((p->k_pages == nullptr) != (p->k_proj == nullptr) || (p->v_pages == nullptr) != (p->v_proj == nullptr))
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: a pool and its projection go together", who);
  if (!p->k_pages && !p->v_pages) return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: nothing to insert", who);
  const int es = p->dtype == AXL_F32 ? 4 : 2;
  const int64_t m = 16 / es;
  if (p->head_dim % m != 0)
    return set_error(AXL_ERR_UNSUPPORTED, "%s: head_dim %d is not a multiple of %d", who, p->head_dim, (int)m);
  if (p->k_proj_batch_stride % m || p->k_proj_head_stride % m || p->v_proj_batch_stride % m ||
      p->v_proj_head_stride % m || !aligned16(p->k_pages) || !aligned16(p->v_pages) ||
      !aligned16(p->k_proj) || !aligned16(p->v_proj))
    return set_error(AXL_ERR_UNSUPPORTED, "%s: rows must be 16-byte aligned", who);
  return launch_page_insert(*p, (hipStream_t)stream);
}

const char* axl_last_error(void) { return g_last_error; }

int axl_abi_version(void) { return AXL_ATTN_ABI_VERSION; }

int axl_flash_fwd(const AxlFlashFwdParams* p, void* stream) {
  if (!p) return set_error(AXL_ERR_INVALID_ARGUMENT, "axl_flash_fwd: params is NULL");
  int rc = check_flash_shapes("axl_flash_fwd", p->batch, p->q_len, p->kv_len, p->num_q_heads,
                              p->num_kv_heads, p->head_dim, p->dtype, p->mask_kind,
                              p->sliding_window, p->softmax_scale, p->segment_ids);
  if (rc != AXL_OK) return rc;
  if (!p->q || !p->k || !p->v || !p->out)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "axl_flash_fwd: NULL tensor pointer");
  const int eb = p->dtype == AXL_F32 ? 4 : 2;
  if (!aligned16(p->q) || !aligned16(p->k) || !aligned16(p->v) || !aligned16(p->out) ||
      !strides_ok(p->q_strides, eb) || !strides_ok(p->k_strides, eb) ||
      !strides_ok(p->v_strides, eb) || !strides_ok(p->out_strides, eb))
    return set_error(AXL_ERR_UNSUPPORTED, "axl_flash_fwd: tensors must be 16-byte aligned rows");
  if (p->segment_ids && !aligned16(p->segment_ids))
    return set_error(AXL_ERR_UNSUPPORTED, "axl_flash_fwd: segment_ids must be 16-byte aligned");
  rc = check_aux("axl_flash_fwd", p->aux, p->batch, p->num_q_heads, p->q_len, p->kv_len);
  if (rc != AXL_OK) return rc;
  rc = check_odd_head_dim("axl_flash_fwd", p->head_dim, p->aux.bias || p->aux.dropout_mask,
                          {&p->q_strides, &p->k_strides, &p->v_strides, &p->out_strides});
  if (rc != AXL_OK) return rc;
  return launch_flash_fwd(*p, (hipStream_t)stream);
}

size_t axl_flash_bwd_workspace_bytes(const AxlFlashBwdParams* p) {
  if (!p) return 0;
  return flash_bwd_workspace_bytes(*p);
}


int axl_flash_bwd(const AxlFlashBwdParams* p, void* stream) {
  return axl_flash_bwd_phases(p, AXL_BWD_DELTA | AXL_BWD_DKDV | AXL_BWD_DQ, stream);
}

int axl_flash_bwd_phases(const AxlFlashBwdParams* p, int phases, void* stream) {
  if (!p) return set_error(AXL_ERR_INVALID_ARGUMENT, "axl_flash_bwd: params is NULL");
  if (phases <= 0 || phases > 7)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "axl_flash_bwd: phases must be in 1..7");
  int rc = check_flash_shapes("axl_flash_bwd", p->batch, p->q_len, p->kv_len, p->num_q_heads,
                              p->num_kv_heads, p->head_dim, p->dtype, p->mask_kind,
                              p->sliding_window, p->softmax_scale, p->segment_ids);
  if (rc != AXL_OK) return rc;
  if (!p->q || !p->k || !p->v || !p->out || !p->d_out || !p->lse || !p->dq || !p->dk || !p->dv)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "axl_flash_bwd: NULL tensor pointer");
  const int eb = p->dtype == AXL_F32 ? 4 : 2;
  const void* ptrs[] = {p->q, p->k, p->v, p->out, p->d_out, p->dq, p->dk, p->dv};
  for (const void* x : ptrs)
    if (!aligned16(x))
      return set_error(AXL_ERR_UNSUPPORTED, "axl_flash_bwd: tensors must be 16-byte aligned");
  const AxlStrides* ss[] = {&p->q_strides,     &p->k_strides,  &p->v_strides,  &p->out_strides,
                            &p->d_out_strides, &p->dq_strides, &p->dk_strides, &p->dv_strides};
  for (const AxlStrides* s : ss)
    if (!strides_ok(*s, eb))
      return set_error(AXL_ERR_UNSUPPORTED, "axl_flash_bwd: rows must be 16-byte aligned");
  if (p->segment_ids && !aligned16(p->segment_ids))
    return set_error(AXL_ERR_UNSUPPORTED, "axl_flash_bwd: segment_ids must be 16-byte aligned");
  rc = check_aux("axl_flash_bwd", p->aux, p->batch, p->num_q_heads, p->q_len, p->kv_len);
  if (rc != AXL_OK) return rc;
  rc = check_odd_head_dim("axl_flash_bwd", p->head_dim, p->aux.bias || p->aux.dropout_mask,
                          {&p->q_strides, &p->k_strides, &p->v_strides, &p->out_strides, &p->d_out_strides,
                           &p->dq_strides, &p->dk_strides, &p->dv_strides});
  if (rc != AXL_OK) return rc;
  const size_t need = flash_bwd_workspace_bytes(*p);
  if (!p->workspace || p->workspace_bytes < need || !aligned16(p->workspace))
    return set_error(AXL_ERR_WORKSPACE, "axl_flash_bwd: workspace needs %zu bytes, 16-byte aligned (got %zu)",
                     need, p->workspace ? p->workspace_bytes : (size_t)0);
  if (p->d_logit_sink && !p->logit_sink)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "axl_flash_bwd: d_logit_sink without logit_sink");
  return launch_flash_bwd(*p, phases, (hipStream_t)stream);
}

static int check_decode_common(const char* who, int batch, int hq, int hkv, int d, int dtype,
                               float scale, const AxlDecodeBias& bias) {
  if (batch <= 0 || hq <= 0 || hkv <= 0 || d <= 0)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: non-positive dimension", who);
  if (hq % hkv != 0)
    return set_error(AXL_ERR_INVALID_ARGUMENT,
                     "%s: num_q_heads %d is not divisible by num_kv_heads %d", who, hq, hkv);
  if (!(scale > 0.f) || !std::isfinite(scale))
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: softmax_scale must be finite and > 0", who);
  if (dtype != AXL_BF16 && dtype != AXL_F16 && dtype != AXL_F32)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: unknown dtype %d", who, dtype);
  if (d > 128 || d % 8 != 0)
    return set_error(AXL_ERR_UNSUPPORTED, "%s: head_dim %d (supported: multiples of 8 up to 128)", who, d);
  if (bias.bias) {
    if (bias.dtype != AXL_BF16 && bias.dtype != AXL_F32)
      return set_error(AXL_ERR_UNSUPPORTED, "%s: bias dtype %d (supported: bf16, fp32)", who, bias.dtype);
    if (bias.batch_stride < 0 || bias.head_stride < 0)
      return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: bias strides must be >= 0", who);
    if (reinterpret_cast<uintptr_t>(bias.bias) % (bias.dtype == AXL_F32 ? 4 : 2))
      return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: bias is not aligned to its element type", who);
  }
  return AXL_OK;
}

size_t axl_paged_decode_workspace_bytes(const AxlPagedDecodeParams* p) {
  if (!p) return 0;
  return paged_decode_workspace_bytes(*p);
}

// Everything axl_paged_decode checks except the workspace.
static int check_paged_decode(const char* who, const AxlPagedDecodeParams* p) {
  if (!p) return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: params is NULL", who);
  int rc = check_decode_common(who, p->batch, p->num_q_heads, p->num_kv_heads, p->head_dim, p->dtype,
                               p->softmax_scale, p->bias);
  if (rc != AXL_OK) return rc;
  if (p->num_pages <= 0 || p->page_size <= 0 || p->pages_per_seq <= 0)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: non-positive page geometry", who);
  if (!p->q || !p->k_pages || !p->v_pages || !p->page_tables || !p->lengths || !p->out)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", who);
  if (p->page_size < 16 || (p->page_size & (p->page_size - 1)) != 0)
    return set_error(AXL_ERR_UNSUPPORTED, "%s: page_size %d (supported: 16 times a power of two)", who, p->page_size);
  if ((int64_t)p->page_size * p->pages_per_seq > (int64_t)1 << 30)
    return set_error(AXL_ERR_UNSUPPORTED, "%s: page_size * pages_per_seq above 2^30", who);
  if (!aligned16(p->q) || !aligned16(p->k_pages) || !aligned16(p->v_pages) || !aligned16(p->out))
    return set_error(AXL_ERR_UNSUPPORTED, "%s: tensors must be 16-byte aligned", who);
  return AXL_OK;
}

int axl_paged_decode_static(const AxlPagedDecodeParams* p, void* stream) {
  const int rc = check_paged_decode("axl_paged_decode_static", p);
  if (rc != AXL_OK) return rc;
  return launch_paged_decode_static(*p, (hipStream_t)stream);
}

int axl_paged_decode(const AxlPagedDecodeParams* p, void* stream) {
  const int rc = check_paged_decode("axl_paged_decode", p);
  if (rc != AXL_OK) return rc;
  const size_t need = paged_decode_workspace_bytes(*p);
  if (!p->workspace || p->workspace_bytes < need || !aligned16(p->workspace))
    return set_error(AXL_ERR_WORKSPACE, "axl_paged_decode: workspace needs %zu bytes, got %zu",
                     need, p->workspace ? p->workspace_bytes : (size_t)0);
  return launch_paged_decode(*p, (hipStream_t)stream);
}

size_t axl_decode_workspace_bytes(const AxlDecodeParams* p) {
  if (!p) return 0;
  return decode_workspace_bytes(*p);
}

int axl_decode(const AxlDecodeParams* p, void* stream) {
  if (!p) return set_error(AXL_ERR_INVALID_ARGUMENT, "axl_decode: params is NULL");
  int rc = check_decode_common("axl_decode", p->batch, p->num_q_heads, p->num_kv_heads,
                               p->head_dim, p->dtype, p->softmax_scale, p->bias);
  if (rc != AXL_OK) return rc;
  if (p->kv_len <= 0) return set_error(AXL_ERR_INVALID_ARGUMENT, "axl_decode: kv_len <= 0");
  if (!p->q || !p->k || !p->v || !p->lengths || !p->out)
    return set_error(AXL_ERR_INVALID_ARGUMENT, "axl_decode: NULL tensor pointer");
  if (!aligned16(p->q) || !aligned16(p->k) || !aligned16(p->v) || !aligned16(p->out) ||
      !strides_ok(p->k_strides, p->dtype == AXL_F32 ? 4 : 2) ||
      !strides_ok(p->v_strides, p->dtype == AXL_F32 ? 4 : 2))
    return set_error(AXL_ERR_UNSUPPORTED, "axl_decode: tensors must be 16-byte aligned rows");
  const size_t need = decode_workspace_bytes(*p);
  if (!p->workspace || p->workspace_bytes < need || !aligned16(p->workspace))
    return set_error(AXL_ERR_WORKSPACE, "axl_decode: workspace needs %zu bytes, got %zu", need,
                     p->workspace ? p->workspace_bytes : (size_t)0);
  return launch_decode(*p, (hipStream_t)stream);
}

}  // extern "C"
