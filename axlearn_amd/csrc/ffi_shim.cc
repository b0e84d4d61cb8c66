// XLA FFI handlers over the C ABI of libaxl_attn_hip.so (include/axl_attn.h): the custom calls that
// JAX-on-ROCm reaches through jax.ffi.ffi_call.  One handler per entry point:
//
//   AxlFlashFwd        -> axl_flash_fwd         (gpu_attention.py:293-425, pallas_call(mha_forward))
//   AxlFlashBwd        -> axl_flash_bwd         (gpu_attention.py:621-786, `_mha_backward`)
//   AxlDecode          -> axl_decode            (gpu_decoding.py:192-283)
//   AxlPagedDecode     -> axl_paged_decode      (gpu_paged_attention.py:164-296)
//   AxlPagedKvInsert   -> axl_paged_kv_insert   (kv_cache/paged_kv_cache_gpu_kernel.py:36-60)
//
// The reference has no jax.ffi usage of its own (its kernels are Pallas); these handlers are what a
// maintainer adds next to axlearn/common/flash_attention/gpu_attention.py.  The Python side
// (registration, ffi_call wrappers, custom_vjp with the `flash_residuals` tags) is
// axlearn_amd/flash_attention/jax_ffi.py.
//
// Build (not part of the default `make`: the header ships with jaxlib, which this repository's
// environment does not have):
//   hipcc -O2 -std=c++17 -fPIC -shared -I$(python -c 'import jax; print(jax.ffi.include_dir())')
//         -I../../include ffi_shim.cc -L.. -laxl_attn_hip -o ../libaxl_attn_ffi.so
// Here the file is compiled, and its handlers are run by the tests, against a stand-in for that header
// which keeps the names and accessors this file uses (tests/xla_ffi_stand_in/).
//
// Conventions.  Every buffer is a device buffer owned by XLA; the library allocates nothing, so the
// workspaces are extra RESULTS of the custom call (XLA allocates them, the Python wrapper drops
// them).  XLA FFI has no optional operands: an absent segment_ids / logit_sink / bias / dropout mask
// / q_pos_offsets is passed as a zero-element buffer.  Layouts are the default row-major ones, so
// strides are derived from the dimensions.  Scalars travel as attributes.
#include <cstdint>
#include <string>

#include <hip/hip_runtime.h>

#include "axl_attn.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

ffi::Error Fail(const char* who, int rc) {
  return ffi::Error(rc == AXL_ERR_UNSUPPORTED ? ffi::ErrorCode::kUnimplemented : ffi::ErrorCode::kInvalidArgument,
                    std::string(who) + ": " + axl_last_error());
}

int DtypeOf(ffi::DataType t) {
  switch (t) {
    case ffi::DataType::BF16: return AXL_BF16;
    case ffi::DataType::F16: return AXL_F16;
    case ffi::DataType::F32: return AXL_F32;
    default: return -1;
  }
}

// Strides of a dense row-major [batch, seq, heads, head_dim] buffer, in elements.
AxlStrides Dense4(ffi::Span<const int64_t> d) { return AxlStrides{d[1] * d[2] * d[3], d[2] * d[3], d[3]}; }

template <typename T>
const T* OrNull(const ffi::AnyBuffer& b) {
  return b.element_count() == 0 ? nullptr : static_cast<const T*>(b.untyped_data());
}

// bias [B|1, Hq|1, T, S] and dropout mask [B, Hq, T, S] (uint8 / pred, nonzero = dropped).
ffi::Error FillAux(const char* who, const ffi::AnyBuffer& bias, const ffi::AnyBuffer& drop, float rate, AxlAttnAux* aux) {
  *aux = AxlAttnAux{};
  if (bias.element_count() != 0) {
    auto d = bias.dimensions();
    if (d.size() != 4) return ffi::Error(ffi::ErrorCode::kInvalidArgument, std::string(who) + ": bias must be 4-d");
    const int dt = DtypeOf(bias.element_type());
    if (dt != AXL_BF16 && dt != AXL_F32)
      return ffi::Error(ffi::ErrorCode::kUnimplemented, std::string(who) + ": bias must be bf16 or f32");
    aux->bias = bias.untyped_data();
    aux->bias_dtype = dt;
    aux->bias_row_stride = d[3];
    aux->bias_head_stride = d[1] == 1 ? 0 : d[2] * d[3];
    aux->bias_batch_stride = d[0] == 1 ? 0 : d[1] * d[2] * d[3];
  }
  if (drop.element_count() != 0) {
    auto d = drop.dimensions();
    if (d.size() != 4) return ffi::Error(ffi::ErrorCode::kInvalidArgument, std::string(who) + ": dropout mask must be 4-d");
    aux->dropout_mask = static_cast<const uint8_t*>(drop.untyped_data());
    aux->dropout_rate = rate;
    aux->drop_row_stride = d[3];
    aux->drop_head_stride = d[2] * d[3];
    aux->drop_batch_stride = d[1] * d[2] * d[3];
  }
  return ffi::Error::Success();
}

// ---------------------------------------------------------------------------------------------
// Forward.  Operands: q [B,T,Hq,D], k, v [B,S,Hkv,D], segment_ids [B,T] s32 | [0], logit_sink [Hq]
// f32 | [0], bias | [0], dropout_mask | [0], q_pos_offsets [B] s32 | [0].  Results: out [B,T,Hq,D],
// lse [B,Hq,T] f32 (the residuals the Python side tags `flash_residuals`).
// ---------------------------------------------------------------------------------------------
ffi::Error FlashFwd(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer segment_ids,
                    ffi::AnyBuffer logit_sink, ffi::AnyBuffer bias, ffi::AnyBuffer dropout_mask,
                    ffi::AnyBuffer q_pos_offsets, ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> lse,
                    float softmax_scale, int32_t mask_kind, int32_t sliding_window, int32_t q_pos_offset,
                    float dropout_rate) {
  auto qd = q.dimensions(), kd = k.dimensions();
  if (qd.size() != 4 || kd.size() != 4)
    return ffi::Error(ffi::ErrorCode::kInvalidArgument, "axl_flash_fwd: q, k, v must be [batch, seq, heads, head_dim]");
  AxlFlashFwdParams p{};
  p.q = q.untyped_data(); p.k = k.untyped_data(); p.v = v.untyped_data();
  p.out = out->untyped_data();
  p.lse = static_cast<float*>(lse->untyped_data());
  p.segment_ids = OrNull<int32_t>(segment_ids);
  p.q_strides = Dense4(qd); p.k_strides = Dense4(kd); p.v_strides = Dense4(v.dimensions());
  p.out_strides = Dense4(out->dimensions());
  p.batch = (int32_t)qd[0]; p.q_len = (int32_t)qd[1]; p.num_q_heads = (int32_t)qd[2]; p.head_dim = (int32_t)qd[3];
  p.kv_len = (int32_t)kd[1]; p.num_kv_heads = (int32_t)kd[2];
  p.dtype = DtypeOf(q.element_type());
  p.mask_kind = mask_kind; p.sliding_window = sliding_window; p.q_pos_offset = q_pos_offset;
  p.softmax_scale = softmax_scale;
  p.logit_sink = OrNull<float>(logit_sink);
  p.q_pos_offsets = OrNull<int32_t>(q_pos_offsets);
  if (auto e = FillAux("axl_flash_fwd", bias, dropout_mask, dropout_rate, &p.aux); e.failure()) return e;
  const int rc = axl_flash_fwd(&p, stream);
  return rc == AXL_OK ? ffi::Error::Success() : Fail("axl_flash_fwd", rc);
}

// ---------------------------------------------------------------------------------------------
// Backward.  Operands: q, k, v, out, d_out, lse, then the optional ones of the forward (segment_ids,
// logit_sink, bias, dropout_mask).  Results: dq, dk [B,S,Hkv,D], dv, d_logit_sink [Hq] f32 | [0], and
// the workspace (u8, `workspace_bytes` as computed by axl_flash_bwd_workspace_bytes on the Python
// side through the same library; the wrapper discards it).
// ---------------------------------------------------------------------------------------------
ffi::Error FlashBwd(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer out,
                    ffi::AnyBuffer d_out, ffi::AnyBuffer lse, ffi::AnyBuffer segment_ids, ffi::AnyBuffer logit_sink,
                    ffi::AnyBuffer bias, ffi::AnyBuffer dropout_mask, ffi::Result<ffi::AnyBuffer> dq,
                    ffi::Result<ffi::AnyBuffer> dk, ffi::Result<ffi::AnyBuffer> dv,
                    ffi::Result<ffi::AnyBuffer> d_logit_sink, ffi::Result<ffi::AnyBuffer> workspace,
                    float softmax_scale, int32_t mask_kind, int32_t sliding_window, int32_t q_pos_offset,
                    float dropout_rate, int32_t flags) {
  auto qd = q.dimensions(), kd = k.dimensions();
  if (qd.size() != 4 || kd.size() != 4)
    return ffi::Error(ffi::ErrorCode::kInvalidArgument, "axl_flash_bwd: q, k, v must be [batch, seq, heads, head_dim]");
  AxlFlashBwdParams p{};
  p.q = q.untyped_data(); p.k = k.untyped_data(); p.v = v.untyped_data();
  p.out = out.untyped_data(); p.d_out = d_out.untyped_data();
  p.lse = static_cast<const float*>(lse.untyped_data());
  p.dq = dq->untyped_data(); p.dk = dk->untyped_data(); p.dv = dv->untyped_data();
  p.segment_ids = OrNull<int32_t>(segment_ids);
  p.q_strides = Dense4(qd); p.k_strides = Dense4(kd); p.v_strides = Dense4(v.dimensions());
  p.out_strides = Dense4(out.dimensions()); p.d_out_strides = Dense4(d_out.dimensions());
  p.dq_strides = Dense4(dq->dimensions()); p.dk_strides = Dense4(dk->dimensions());
  p.dv_strides = Dense4(dv->dimensions());
  p.batch = (int32_t)qd[0]; p.q_len = (int32_t)qd[1]; p.num_q_heads = (int32_t)qd[2]; p.head_dim = (int32_t)qd[3];
  p.kv_len = (int32_t)kd[1]; p.num_kv_heads = (int32_t)kd[2];
  p.dtype = DtypeOf(q.element_type());
  p.mask_kind = mask_kind; p.sliding_window = sliding_window; p.q_pos_offset = q_pos_offset;
  p.softmax_scale = softmax_scale;
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  p.logit_sink = OrNull<float>(logit_sink);
  p.d_logit_sink = d_logit_sink->element_count() == 0 ? nullptr : static_cast<float*>(d_logit_sink->untyped_data());
  p.flags = flags;
  if (auto e = FillAux("axl_flash_bwd", bias, dropout_mask, dropout_rate, &p.aux); e.failure()) return e;
  const int rc = axl_flash_bwd(&p, stream);
  return rc == AXL_OK ? ffi::Error::Success() : Fail("axl_flash_bwd", rc);
}

// Decode bias operand: [B|1, Hq|1, S] bf16 / f32, or an empty buffer for none.
ffi::Error FillDecodeBias(const char* who, const ffi::AnyBuffer& bias, AxlDecodeBias* out) {
  *out = AxlDecodeBias{};
  if (bias.element_count() == 0) return ffi::Error::Success();
  auto d = bias.dimensions();
  if (d.size() != 3) return ffi::Error(ffi::ErrorCode::kInvalidArgument, std::string(who) + ": bias must be [B|1, Hq|1, S]");
  const int dt = DtypeOf(bias.element_type());
  if (dt != AXL_BF16 && dt != AXL_F32)
    return ffi::Error(ffi::ErrorCode::kUnimplemented, std::string(who) + ": bias must be bf16 or f32");
  out->bias = bias.untyped_data();
  out->dtype = dt;
  out->head_stride = d[1] == 1 ? 0 : d[2];
  out->batch_stride = d[0] == 1 ? 0 : d[1] * d[2];
  return ffi::Error::Success();
}

// ---------------------------------------------------------------------------------------------
// Contiguous-cache decode.  Operands: q [B,Hq,D], k, v [B,S,Hkv,D], lengths [B] s32, bias [B|1,Hq|1,S]
// | [0].  Results: out [B,Hq,D], workspace (u8, sized by axl_decode_workspace_bytes with the same
// bias presence).
// ---------------------------------------------------------------------------------------------
ffi::Error Decode(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer lengths,
                  ffi::AnyBuffer bias, ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> workspace,
                  float softmax_scale, int32_t sliding_window, int32_t flags) {
  auto qd = q.dimensions(), kd = k.dimensions();
  if (qd.size() != 3 || kd.size() != 4)
    return ffi::Error(ffi::ErrorCode::kInvalidArgument, "axl_decode: q must be [B,Hq,D], k / v [B,S,Hkv,D]");
  AxlDecodeParams p{};
  p.q = q.untyped_data(); p.k = k.untyped_data(); p.v = v.untyped_data();
  p.lengths = static_cast<const int32_t*>(lengths.untyped_data());
  p.out = out->untyped_data();
  p.k_strides = Dense4(kd); p.v_strides = Dense4(v.dimensions());
  p.batch = (int32_t)qd[0]; p.num_q_heads = (int32_t)qd[1]; p.head_dim = (int32_t)qd[2];
  p.kv_len = (int32_t)kd[1]; p.num_kv_heads = (int32_t)kd[2];
  p.dtype = DtypeOf(q.element_type());
  p.sliding_window = sliding_window; p.softmax_scale = softmax_scale;
  p.workspace = workspace->untyped_data(); p.workspace_bytes = workspace->size_bytes();
  // XLA hands out a fresh scratch buffer per call: never AXL_DECODE_WORKSPACE_REUSED.
  p.flags = flags & AXL_DECODE_DETERMINISTIC;
  if (auto e = FillDecodeBias("axl_decode", bias, &p.bias); e.failure()) return e;
  const int rc = axl_decode(&p, stream);
  return rc == AXL_OK ? ffi::Error::Success() : Fail("axl_decode", rc);
}

// ---------------------------------------------------------------------------------------------
// Paged decode.  Operands: q [B,Hq,D], k_pages, v_pages [Hkv,P,page,D], page_tables [B,pps] s32,
// lengths [B] s32, bias [B|1,Hq|1,pps*page] | [0].  Results: out [B,Hq,D], workspace (u8).
// ---------------------------------------------------------------------------------------------
ffi::Error PagedDecode(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k_pages, ffi::AnyBuffer v_pages,
                       ffi::AnyBuffer page_tables, ffi::AnyBuffer lengths, ffi::AnyBuffer bias,
                       ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> workspace, float softmax_scale,
                       int32_t sliding_window, int32_t flags) {
  auto qd = q.dimensions(), pd = k_pages.dimensions(), td = page_tables.dimensions();
  if (qd.size() != 3 || pd.size() != 4 || td.size() != 2)
    return ffi::Error(ffi::ErrorCode::kInvalidArgument,
                      "axl_paged_decode: q must be [B,Hq,D], pools [Hkv,P,page,D], page_tables [B,pps]");
  AxlPagedDecodeParams p{};
  p.q = q.untyped_data(); p.k_pages = k_pages.untyped_data(); p.v_pages = v_pages.untyped_data();
  p.page_tables = static_cast<const int32_t*>(page_tables.untyped_data());
  p.lengths = static_cast<const int32_t*>(lengths.untyped_data());
  p.out = out->untyped_data();
  p.batch = (int32_t)qd[0]; p.num_q_heads = (int32_t)qd[1]; p.head_dim = (int32_t)qd[2];
  p.num_kv_heads = (int32_t)pd[0]; p.num_pages = (int32_t)pd[1]; p.page_size = (int32_t)pd[2];
  p.pages_per_seq = (int32_t)td[1];
  p.dtype = DtypeOf(q.element_type());
  p.sliding_window = sliding_window; p.softmax_scale = softmax_scale;
  p.workspace = workspace->untyped_data(); p.workspace_bytes = workspace->size_bytes();
  p.flags = flags & AXL_DECODE_DETERMINISTIC;
  if (auto e = FillDecodeBias("axl_paged_decode", bias, &p.bias); e.failure()) return e;
  const int rc = axl_paged_decode(&p, stream);
  return rc == AXL_OK ? ffi::Error::Success() : Fail("axl_paged_decode", rc);
}

// ---------------------------------------------------------------------------------------------
// Page insert, in place.  Operands: k_pages, v_pages [Hkv,P,page,D], k_proj, v_proj [Hkv,B,1,D] (the
// kernel layout of paged_kv_cache_gpu_kernel.py:36-60), page_indices [B,pps] s32, key_positions [B]
// or [1] s32.  Results: k_pages, v_pages, declared on the Python side with
// input_output_aliases={0: 0, 1: 1} as the reference's pallas_call does (:57), so XLA normally hands
// the operand's own buffer back as the result; if it could not alias, the pool is copied first.
// ---------------------------------------------------------------------------------------------
ffi::Error PagedKvInsert(hipStream_t stream, ffi::AnyBuffer k_pages, ffi::AnyBuffer v_pages, ffi::AnyBuffer k_proj,
                         ffi::AnyBuffer v_proj, ffi::AnyBuffer page_indices, ffi::AnyBuffer key_positions,
                         ffi::Result<ffi::AnyBuffer> k_out, ffi::Result<ffi::AnyBuffer> v_out) {
  auto pd = k_pages.dimensions(), jd = k_proj.dimensions(), id = page_indices.dimensions();
  if (pd.size() != 4 || jd.size() != 4 || id.size() != 2)
    return ffi::Error(ffi::ErrorCode::kInvalidArgument,
                      "axl_paged_kv_insert: pools [Hkv,P,page,D], projections [Hkv,B,1,D], page_indices [B,pps]");
  if (k_out->untyped_data() != k_pages.untyped_data() &&
      hipMemcpyAsync(k_out->untyped_data(), k_pages.untyped_data(), k_pages.size_bytes(), hipMemcpyDeviceToDevice, stream) != hipSuccess)
    return ffi::Error(ffi::ErrorCode::kInternal, "axl_paged_kv_insert: copying the K pool failed");
  if (v_out->untyped_data() != v_pages.untyped_data() &&
      hipMemcpyAsync(v_out->untyped_data(), v_pages.untyped_data(), v_pages.size_bytes(), hipMemcpyDeviceToDevice, stream) != hipSuccess)
    return ffi::Error(ffi::ErrorCode::kInternal, "axl_paged_kv_insert: copying the V pool failed");
  AxlPageInsertParams p{};
  p.k_pages = k_out->untyped_data(); p.v_pages = v_out->untyped_data();
  p.k_proj = k_proj.untyped_data(); p.v_proj = v_proj.untyped_data();
  p.page_indices = static_cast<const int32_t*>(page_indices.untyped_data());
  p.key_positions = static_cast<const int32_t*>(key_positions.untyped_data());
  // [Hkv, B, 1, D]: element (b, h, :) at b * D + h * B * D
  p.k_proj_batch_stride = p.v_proj_batch_stride = jd[3];
  p.k_proj_head_stride = p.v_proj_head_stride = jd[1] * jd[2] * jd[3];
  p.batch = (int32_t)id[0]; p.pages_per_seq = (int32_t)id[1];
  p.num_kv_heads = (int32_t)pd[0]; p.num_pages = (int32_t)pd[1]; p.page_size = (int32_t)pd[2]; p.head_dim = (int32_t)pd[3];
  p.dtype = DtypeOf(k_pages.element_type());
  p.broadcast_positions = key_positions.element_count() == 1 && id[0] > 1;
  const int rc = axl_paged_kv_insert(&p, stream);
  return rc == AXL_OK ? ffi::Error::Success() : Fail("axl_paged_kv_insert", rc);
}

}  // namespace

// The ABI version of include/axl_attn.h this file was compiled against: the Python side compares it with
// axl_abi_version() of the core library before it registers the handlers (the structures are filled here
// and read there).
extern "C" int axl_ffi_shim_abi_version() { return AXL_ATTN_ABI_VERSION; }

XLA_FFI_DEFINE_HANDLER_SYMBOL(AxlFlashFwd, FlashFwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()  // q
                                  .Arg<ffi::AnyBuffer>()  // k
                                  .Arg<ffi::AnyBuffer>()  // v
                                  .Arg<ffi::AnyBuffer>()  // segment_ids | [0]
                                  .Arg<ffi::AnyBuffer>()  // logit_sink | [0]
                                  .Arg<ffi::AnyBuffer>()  // bias | [0]
                                  .Arg<ffi::AnyBuffer>()  // dropout_mask | [0]
                                  .Arg<ffi::AnyBuffer>()  // q_pos_offsets | [0]
                                  .Ret<ffi::AnyBuffer>()  // out
                                  .Ret<ffi::AnyBuffer>()  // lse
                                  .Attr<float>("softmax_scale")
                                  .Attr<int32_t>("mask_kind")
                                  .Attr<int32_t>("sliding_window")
                                  .Attr<int32_t>("q_pos_offset")
                                  .Attr<float>("dropout_rate"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(AxlFlashBwd, FlashBwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()  // q
                                  .Arg<ffi::AnyBuffer>()  // k
                                  .Arg<ffi::AnyBuffer>()  // v
                                  .Arg<ffi::AnyBuffer>()  // out
                                  .Arg<ffi::AnyBuffer>()  // d_out
                                  .Arg<ffi::AnyBuffer>()  // lse
                                  .Arg<ffi::AnyBuffer>()  // segment_ids | [0]
                                  .Arg<ffi::AnyBuffer>()  // logit_sink | [0]
                                  .Arg<ffi::AnyBuffer>()  // bias | [0]
                                  .Arg<ffi::AnyBuffer>()  // dropout_mask | [0]
                                  .Ret<ffi::AnyBuffer>()  // dq
                                  .Ret<ffi::AnyBuffer>()  // dk
                                  .Ret<ffi::AnyBuffer>()  // dv
                                  .Ret<ffi::AnyBuffer>()  // d_logit_sink | [0]
                                  .Ret<ffi::AnyBuffer>()  // workspace
                                  .Attr<float>("softmax_scale")
                                  .Attr<int32_t>("mask_kind")
                                  .Attr<int32_t>("sliding_window")
                                  .Attr<int32_t>("q_pos_offset")
                                  .Attr<float>("dropout_rate")
                                  .Attr<int32_t>("flags"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(AxlDecode, Decode,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()  // q
                                  .Arg<ffi::AnyBuffer>()  // k
                                  .Arg<ffi::AnyBuffer>()  // v
                                  .Arg<ffi::AnyBuffer>()  // lengths
                                  .Arg<ffi::AnyBuffer>()  // bias | [0]
                                  .Ret<ffi::AnyBuffer>()  // out
                                  .Ret<ffi::AnyBuffer>()  // workspace
                                  .Attr<float>("softmax_scale")
                                  .Attr<int32_t>("sliding_window")
                                  .Attr<int32_t>("flags"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(AxlPagedDecode, PagedDecode,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()  // q
                                  .Arg<ffi::AnyBuffer>()  // k_pages
                                  .Arg<ffi::AnyBuffer>()  // v_pages
                                  .Arg<ffi::AnyBuffer>()  // page_tables
                                  .Arg<ffi::AnyBuffer>()  // lengths
                                  .Arg<ffi::AnyBuffer>()  // bias | [0]
                                  .Ret<ffi::AnyBuffer>()  // out
                                  .Ret<ffi::AnyBuffer>()  // workspace
                                  .Attr<float>("softmax_scale")
                                  .Attr<int32_t>("sliding_window")
                                  .Attr<int32_t>("flags"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(AxlPagedKvInsert, PagedKvInsert,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()  // k_pages
                                  .Arg<ffi::AnyBuffer>()  // v_pages
                                  .Arg<ffi::AnyBuffer>()  // k_proj
                                  .Arg<ffi::AnyBuffer>()  // v_proj
                                  .Arg<ffi::AnyBuffer>()  // page_indices
                                  .Arg<ffi::AnyBuffer>()  // key_positions
                                  .Ret<ffi::AnyBuffer>()  // k_pages (aliased to operand 0)
                                  .Ret<ffi::AnyBuffer>());  // v_pages (aliased to operand 1)
