"""Tensor-level wrappers over the C ABI: allocate outputs/workspace with torch, pass raw pointers.

These are the functions the `BaseFlashAttention`-shaped classes in `axlearn_amd.flash_attention`
call. Inputs must be CUDA(ROCm) tensors; torch is used for device memory and streams only.
"""

from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from axlearn_amd import _lib
from axlearn_amd._lib import (
    MASK_CAUSAL,
    MASK_NONE,
    MASK_SLIDING_WINDOW,
    AxlDecodeBias,
    AxlDecodeParams,
    AxlError,
    AxlFlashBwdParams,
    AxlFlashFwdParams,
    AxlPagedDecodeParams,
    AxlPageInsertParams,
)

__all__ = [
    "MASK_NONE",
    "MASK_CAUSAL",
    "MASK_SLIDING_WINDOW",
    "flash_fwd",
    "flash_bwd",
    "flash_bwd_buffers",
    "flash_bwd_ds_workspace_bytes",
    "default_bwd_workspace_limit",
    "paged_decode",
    "decode",
]


def _require_cuda(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, "all tensors must live on the GPU")
        if dev is not None and t.device != dev:
            raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, f"tensors live on different devices ({dev} and {t.device})")
        dev = t.device


def _bad(msg: str) -> AxlError:
    return AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, msg)


def _want_shape(name: str, t: torch.Tensor, shape) -> None:
    if tuple(t.shape) != tuple(shape):
        raise _bad(f"{name} must have shape {list(shape)}, got {list(t.shape)}")


def _check_qkv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
    """The kernels take every extent from these shapes and read raw pointers: anything that does not
    fit together is rejected here, before a parameter block is built."""
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise _bad(f"q, k, v must be 4-d [batch, seq, heads, head_dim], got {list(q.shape)}, {list(k.shape)}, {list(v.shape)}")
    b, t, hq, d = q.shape
    if k.shape[0] != b or k.shape[3] != d:
        raise _bad(f"k {list(k.shape)} does not match q {list(q.shape)} in batch / head_dim")
    if tuple(v.shape) != tuple(k.shape):
        raise _bad(f"v {list(v.shape)} must have the shape of k {list(k.shape)}")
    hkv = k.shape[2]
    if hkv <= 0 or hq % hkv != 0:
        raise _bad(f"num_q_heads {hq} is not divisible by num_kv_heads {hkv}")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise AxlError(_lib.AXL_ERR_UNSUPPORTED, "q, k, v must share one dtype")
    return b, t, hq, d, k.shape[1], hkv


def _check_segment_ids(segment_ids: Optional[torch.Tensor], b: int, t: int, s: int) -> None:
    if segment_ids is None:
        return
    if t != s:
        raise _bad(f"segment_ids need q_len == kv_len (got {t} vs {s})")
    _want_shape("segment_ids", segment_ids, (b, t))


def _sink(logit_sink: Optional[torch.Tensor], num_heads: int) -> Optional[torch.Tensor]:
    if logit_sink is None:
        return None
    if tuple(logit_sink.shape) != (num_heads,):
        raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, f"logit_sink must have shape [{num_heads}]")
    return logit_sink.detach().to(torch.float32).contiguous()


def _aux(bias, dropout_mask, dropout_rate, b, hq, t, s) -> Tuple[_lib.AxlAttnAux, tuple]:
    """Builds the AxlAttnAux block; returns it with the tensors it points at (keep them alive)."""
    aux = _lib.AxlAttnAux()
    keep = []
    if bias is not None:
        if bias.dim() != 4 or bias.shape[0] not in (1, b) or bias.shape[1] not in (1, hq) or tuple(bias.shape[2:]) != (t, s):
            raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, f"bias must be [{b}|1, {hq}|1, {t}, {s}], got {tuple(bias.shape)}")
        if bias.dtype not in (torch.bfloat16, torch.float32):
            bias = bias.to(torch.float32)
        if bias.stride(-1) != 1:
            bias = bias.contiguous()
        keep.append(bias)
        aux.bias = bias.data_ptr()
        aux.bias_batch_stride = bias.stride(0) if bias.shape[0] > 1 else 0
        aux.bias_head_stride = bias.stride(1) if bias.shape[1] > 1 else 0
        aux.bias_row_stride = bias.stride(2)
        aux.bias_dtype = _lib.dtype_code(bias.dtype)
    if dropout_mask is not None:
        if tuple(dropout_mask.shape) != (b, hq, t, s):
            raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, f"dropout_mask must be [{b}, {hq}, {t}, {s}]")
        if dropout_mask.dtype == torch.bool:
            dropout_mask = dropout_mask.view(torch.uint8) if dropout_mask.is_contiguous() else dropout_mask.to(torch.uint8)
        if dropout_mask.dtype != torch.uint8:
            raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, "dropout_mask must be bool or uint8 (nonzero = dropped)")
        if dropout_mask.stride(-1) != 1:
            dropout_mask = dropout_mask.contiguous()
        keep.append(dropout_mask)
        aux.dropout_mask = dropout_mask.data_ptr()
        aux.drop_batch_stride, aux.drop_head_stride, aux.drop_row_stride = dropout_mask.stride()[:3]
        aux.dropout_rate = float(dropout_rate)
    elif dropout_rate:
        raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, "dropout_rate needs a dropout_mask (the kernels draw no random numbers)")
    return aux, tuple(keep)


def _seg(segment_ids: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    if segment_ids is None:
        return None
    if segment_ids.dtype != torch.int32 or not segment_ids.is_contiguous():
        segment_ids = segment_ids.to(torch.int32).contiguous()
    return segment_ids


def flash_fwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    *,
    softmax_scale: float = 1.0,
    mask_kind: int = MASK_NONE,
    sliding_window: int = 0,
    segment_ids: Optional[torch.Tensor] = None,
    q_pos_offset: int = 0,
    return_lse: bool = True,
    logit_sink: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
    dropout_mask: Optional[torch.Tensor] = None,
    dropout_rate: float = 0.0,
    q_pos_offsets: Optional[torch.Tensor] = None,
):
    """q [B,T,Hq,D], k/v [B,S,Hkv,D] -> (out [B,T,Hq,D], lse [B,Hq,T] fp32 or None).

    q_pos_offsets [B] int32: per-sequence position of query row 0, added to q_pos_offset.
    logit_sink [Hq]: optional per-head sink logit (joins the softmax and lse, carries no value).
    bias [B|1,Hq|1,T,S] bf16/fp32: dense additive logit bias.  dropout_mask [B,Hq,T,S] bool/uint8
    (True = dropped) with dropout_rate: kept probabilities are scaled by 1 / (1 - rate)."""
    b, t, hq, d, s, hkv = _check_qkv(q, k, v)
    _check_segment_ids(segment_ids, b, t, s)
    if q_pos_offsets is not None:
        _want_shape("q_pos_offsets", q_pos_offsets, (b,))
    _require_cuda(q, k, v, segment_ids, logit_sink, bias, dropout_mask, q_pos_offsets)
    lib = _lib.load()
    if q_pos_offsets is not None:
        q_pos_offsets = q_pos_offsets.to(torch.int32).contiguous()
    out = torch.empty((b, t, hq, d), dtype=q.dtype, device=q.device)
    lse = torch.empty((b, hq, t), dtype=torch.float32, device=q.device) if return_lse else None
    seg = _seg(segment_ids)
    sink = _sink(logit_sink, hq)
    aux, _keep = _aux(bias, dropout_mask, dropout_rate, b, hq, t, s)
    p = AxlFlashFwdParams(
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(), out=out.data_ptr(), lse=_lib.ptr(lse),
        segment_ids=_lib.ptr(seg),
        q_strides=_lib.strides4(q), k_strides=_lib.strides4(k), v_strides=_lib.strides4(v),
        out_strides=_lib.strides4(out),
        batch=b, q_len=t, kv_len=s, num_q_heads=hq, num_kv_heads=hkv, head_dim=d,
        dtype=_lib.dtype_code(q.dtype), mask_kind=mask_kind, sliding_window=int(sliding_window),
        q_pos_offset=int(q_pos_offset), softmax_scale=float(softmax_scale),
        logit_sink=_lib.ptr(sink), aux=aux, q_pos_offsets=_lib.ptr(q_pos_offsets),
    )
    _lib.check(lib.axl_flash_fwd(ctypes.byref(p), _lib.current_stream_ptr()))
    return out, lse


def flash_bwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    out: torch.Tensor,
    lse: torch.Tensor,
    d_out: torch.Tensor,
    *,
    softmax_scale: float = 1.0,
    mask_kind: int = MASK_NONE,
    sliding_window: int = 0,
    segment_ids: Optional[torch.Tensor] = None,
    q_pos_offset: int = 0,
    phases: int = 7,
    buffers=None,
    logit_sink: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
    dropout_mask: Optional[torch.Tensor] = None,
    dropout_rate: float = 0.0,
    ds_workspace: Optional[bool] = False,
    ds_workspace_limit: Optional[int] = None,
    ds_slice_kv_heads: int = 0,
):
    """Returns (dq [B,T,Hq,D], dk [B,S,Hkv,D], dv [B,S,Hkv,D]) in the dtype of q, followed by
    d_logit_sink [Hq] fp32 when `logit_sink` (the one the forward was given) is passed.

    `phases` selects a subset of {1: delta, 2: dK/dV, 4: dQ} (timing / profiling only); `buffers`
    = (dq, dk, dv, workspace) reuses caller-provided outputs instead of allocating.  bias,
    dropout_mask and dropout_rate must be the ones the forward was given (the bias gets no gradient,
    as in gpu_attention.py:786).  `ds_workspace=True` (AXL_BWD_DS_WORKSPACE; causal or sliding-window
    attention over equal lengths without offsets, bias or dropout; ignored otherwise) keeps dS in a
    larger workspace instead of recomputing it for dq; with `ds_slice_kv_heads=n` the workspace holds
    the dS of n kv heads at a time and the two kernels run slice after slice
    (AXL_BWD_DS_SLICE_KV_HEADS).  `ds_workspace=None` decides by size (`select_ds_slice`): the dS
    workspace is used when that path applies and fits `ds_workspace_limit` bytes (default:
    `default_bwd_workspace_limit`, a sixteenth of the device's memory), whole or in slices of kv
    heads that still fill the GPU."""
    b, t, hq, d, s, hkv = _check_qkv(q, k, v)
    _check_segment_ids(segment_ids, b, t, s)
    if ds_workspace is None:
        ds_workspace, ds_slice_kv_heads = False, 0
        if phases == 7 and bias is None and dropout_mask is None and q_pos_offset == 0:
            ds_workspace, ds_slice_kv_heads = select_ds_slice(q, k, mask_kind=mask_kind, segment_ids=segment_ids,
                                                              limit=ds_workspace_limit)
    _want_shape("out", out, q.shape)
    _want_shape("d_out", d_out, q.shape)
    _want_shape("lse", lse, (b, hq, t))
    if out.dtype != q.dtype or d_out.dtype != q.dtype:
        raise AxlError(_lib.AXL_ERR_UNSUPPORTED, "out and d_out must have the dtype of q")
    ws = None
    if buffers is not None:
        dq, dk, dv, ws = buffers
        _want_shape("buffers dq", dq, q.shape)
        _want_shape("buffers dk", dk, k.shape)
        _want_shape("buffers dv", dv, v.shape)
        if dq.dtype != q.dtype or dk.dtype != q.dtype or dv.dtype != q.dtype:
            raise AxlError(_lib.AXL_ERR_UNSUPPORTED, "buffers dq, dk, dv must have the dtype of q")
    _require_cuda(q, k, v, out, lse, d_out, segment_ids, logit_sink, bias, dropout_mask,
                  *(buffers if buffers is not None else ()))
    lib = _lib.load()
    if buffers is None:
        dq = torch.empty((b, t, hq, d), dtype=q.dtype, device=q.device)
        dk = torch.empty((b, s, hkv, d), dtype=k.dtype, device=q.device)
        dv = torch.empty((b, s, hkv, d), dtype=v.dtype, device=q.device)
    seg = _seg(segment_ids)
    if lse.dtype != torch.float32 or not lse.is_contiguous():
        raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, "lse must be contiguous float32 [B,Hq,T]")
    sink = _sink(logit_sink, hq)
    d_sink = torch.empty((hq,), dtype=torch.float32, device=q.device) if sink is not None else None
    aux, _keep = _aux(bias, dropout_mask, dropout_rate, b, hq, t, s)
    p = AxlFlashBwdParams(
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(), out=out.data_ptr(),
        d_out=d_out.data_ptr(), lse=lse.data_ptr(), dq=dq.data_ptr(), dk=dk.data_ptr(),
        dv=dv.data_ptr(), segment_ids=_lib.ptr(seg),
        q_strides=_lib.strides4(q), k_strides=_lib.strides4(k), v_strides=_lib.strides4(v),
        out_strides=_lib.strides4(out), d_out_strides=_lib.strides4(d_out),
        dq_strides=_lib.strides4(dq), dk_strides=_lib.strides4(dk), dv_strides=_lib.strides4(dv),
        batch=b, q_len=t, kv_len=s, num_q_heads=hq, num_kv_heads=hkv, head_dim=d,
        dtype=_lib.dtype_code(q.dtype), mask_kind=mask_kind, sliding_window=int(sliding_window),
        q_pos_offset=int(q_pos_offset), softmax_scale=float(softmax_scale),
        workspace=None, workspace_bytes=0, logit_sink=_lib.ptr(sink), d_logit_sink=_lib.ptr(d_sink),
        aux=aux, flags=_bwd_flags(ds_workspace, ds_slice_kv_heads),
    )
    need = int(lib.axl_flash_bwd_workspace_bytes(ctypes.byref(p)))
    if ws is None:
        ws = torch.empty((max(need, 256),), dtype=torch.uint8, device=q.device)
    elif ws.numel() * ws.element_size() < need:
        raise AxlError(_lib.AXL_ERR_WORKSPACE, f"buffers workspace holds {ws.numel() * ws.element_size()} bytes, {need} needed")
    p.workspace = ws.data_ptr()
    p.workspace_bytes = ws.numel() * ws.element_size()
    _lib.check(lib.axl_flash_bwd_phases(ctypes.byref(p), int(phases), _lib.current_stream_ptr()))
    if sink is not None:
        return dq, dk, dv, d_sink
    return dq, dk, dv


def _bwd_flags(ds_workspace: bool, ds_slice_kv_heads: int = 0) -> int:
    if not ds_workspace:
        return 0
    if not 0 <= int(ds_slice_kv_heads) < 65536:
        raise _bad(f"ds_slice_kv_heads must be in [0, 65535], got {ds_slice_kv_heads}")
    return _lib.BWD_DS_WORKSPACE | (int(ds_slice_kv_heads) << 8)  # AXL_BWD_DS_SLICE_KV_HEADS(n)


def flash_bwd_buffers(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, mask_kind: int = MASK_NONE,
                      ds_workspace: bool = False, segment_ids: Optional[torch.Tensor] = None,
                      ds_slice_kv_heads: int = 0):
    """Pre-allocates (dq, dk, dv, workspace) for repeated `flash_bwd(..., buffers=...)` calls.

    The workspace holds delta and the scaled lse (fp32 [B,Hq,T] each); with `segment_ids` (the ones the
    calls will pass) also the table of id ranges per 32 rows; with `ds_workspace=True` and a causal or
    sliding-window `mask_kind` (equal lengths, no offsets / bias / dropout) also dS, about T*S bytes per
    (batch, head), for `flash_bwd(..., ds_workspace=True)` - of `ds_slice_kv_heads` kv heads at a time if that
    is given (the calls must pass the same number)."""
    b, t, hq, d = q.shape
    p = AxlFlashBwdParams(batch=b, q_len=t, kv_len=k.shape[1], num_q_heads=hq, num_kv_heads=k.shape[2],
                          head_dim=d, dtype=_lib.dtype_code(q.dtype), mask_kind=mask_kind,
                          segment_ids=_lib.ptr(_seg(segment_ids)),
                          flags=_bwd_flags(ds_workspace, ds_slice_kv_heads))
    nbytes = int(_lib.load().axl_flash_bwd_workspace_bytes(ctypes.byref(p)))
    ws = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=q.device)
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), ws


def flash_bwd_ds_workspace_bytes(q: torch.Tensor, k: torch.Tensor, *, mask_kind: int,
                                 segment_ids: Optional[torch.Tensor] = None,
                                 ds_slice_kv_heads: int = 0) -> Tuple[int, int]:
    """(bytes with AXL_BWD_DS_WORKSPACE, bytes without) of backward workspace for these shapes and
    this mask; the two are equal where the dS-workspace path does not apply (the flag is ignored).
    `ds_slice_kv_heads`: with the dS of that many kv heads at a time (0: all)."""
    b, t, hq, d = q.shape
    p = AxlFlashBwdParams(batch=b, q_len=t, kv_len=k.shape[1], num_q_heads=hq, num_kv_heads=k.shape[2],
                          head_dim=d, dtype=_lib.dtype_code(q.dtype), mask_kind=mask_kind,
                          segment_ids=None if segment_ids is None else 256,
                          flags=_bwd_flags(True, ds_slice_kv_heads))
    lib = _lib.load()
    with_ds = int(lib.axl_flash_bwd_workspace_bytes(ctypes.byref(p)))
    p.flags = 0
    return with_ds, int(lib.axl_flash_bwd_workspace_bytes(ctypes.byref(p)))


def default_bwd_workspace_limit(device) -> int:
    """Transient bytes the backward may take for dS when the caller states no limit: a sixteenth of the
    device's memory (18 GB of an MI355X's 288 GB)."""
    return torch.cuda.get_device_properties(device).total_memory // 16


def select_ds_slice(q: torch.Tensor, k: torch.Tensor, *, mask_kind: int,
                    segment_ids: Optional[torch.Tensor] = None, limit: Optional[int] = None) -> Tuple[bool, int]:
    """The backward's default policy, as (ds_workspace, ds_slice_kv_heads): keep dS in the workspace (5
    executed GEMMs instead of 7) when that path applies to these shapes and its workspace fits `limit`
    bytes - whole (slice 0), or of as many kv heads at a time as fit, provided a slice still gives every
    CU a dK/dV workgroup (batch * heads * kv_len / 256 of them under a causal mask, twice that under a
    window); else the recomputing pair."""
    with_ds, without = flash_bwd_ds_workspace_bytes(q, k, mask_kind=mask_kind, segment_ids=segment_ids)
    if with_ds == without:
        return False, 0
    if limit is None:
        limit = default_bwd_workspace_limit(q.device)
    if with_ds <= int(limit):
        return True, 0
    b, hkv, s = q.shape[0], k.shape[2], k.shape[1]
    heads = min(hkv - 1, (int(limit) - without) * hkv // (with_ds - without) + 1)   # kv heads whose dS fits
    while heads >= 1 and flash_bwd_ds_workspace_bytes(q, k, mask_kind=mask_kind, segment_ids=segment_ids,
                                                      ds_slice_kv_heads=heads)[0] > int(limit):
        heads -= 1
    per_head = b * (s // 128) // (2 if mask_kind == MASK_CAUSAL else 1)   # dK/dV workgroups per kv head
    cus = torch.cuda.get_device_properties(q.device).multi_processor_count
    if heads < 1 or heads * per_head < cus:
        return False, 0
    return True, int(heads)


def select_ds_workspace(q: torch.Tensor, k: torch.Tensor, *, mask_kind: int,
                        segment_ids: Optional[torch.Tensor] = None, limit: Optional[int] = None) -> bool:
    """Whether `select_ds_slice` takes the dS workspace for these shapes (whole or in slices)."""
    return select_ds_slice(q, k, mask_kind=mask_kind, segment_ids=segment_ids, limit=limit)[0]


def _decode_flags(deterministic: bool, workspace_reused: bool) -> int:
    return (_lib.DECODE_DETERMINISTIC if deterministic else 0) | (_lib.DECODE_WORKSPACE_REUSED if workspace_reused else 0)


def _check_decode_out_ws(q, out, workspace):
    if out is not None:
        _want_shape("out", out, q.shape)
        if out.dtype != q.dtype or not out.is_contiguous():
            raise _bad("out must be contiguous and have the dtype of q")
    if workspace is not None and (workspace.dtype != torch.uint8 or not workspace.is_contiguous()):
        raise _bad("workspace must be a contiguous uint8 tensor")


def _decode_bias(bias: Optional[torch.Tensor], b: int, hq: int, kv_len: int):
    """The AxlDecodeBias block for a bias `[B|1, Hq|1, kv_len]`; returns it with the tensor it points at."""
    blk = AxlDecodeBias()
    if bias is None:
        return blk, None
    if bias.dim() != 3 or bias.shape[0] not in (1, b) or bias.shape[1] not in (1, hq) or bias.shape[2] != kv_len:
        raise _bad(f"bias must be [{b}|1, {hq}|1, {kv_len}], got {list(bias.shape)}")
    if bias.dtype not in (torch.bfloat16, torch.float32):
        bias = bias.to(torch.float32)
    if bias.stride(-1) != 1:
        bias = bias.contiguous()
    blk.bias = bias.data_ptr()
    blk.batch_stride = bias.stride(0) if bias.shape[0] > 1 else 0
    blk.head_stride = bias.stride(1) if bias.shape[1] > 1 else 0
    blk.dtype = _lib.dtype_code(bias.dtype)
    return blk, bias


def paged_decode(
    q: torch.Tensor,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    page_tables: torch.Tensor,
    lengths: torch.Tensor,
    *,
    softmax_scale: float = 1.0,
    sliding_window: int = -1,
    workspace: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    deterministic: bool = False,
    workspace_reused: bool = False,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """q [B,Hq,D]; pools [Hkv,P,page,D]; page_tables [B,pps] int32; lengths [B] int32 -> [B,Hq,D].

    Lengths are clamped to [0, pps * page]; a sequence of length 0 yields zeros.  `deterministic`
    fixes the work decomposition (bit-reproducible); `workspace_reused` promises that `workspace` was
    last touched by an earlier decode call (skips the launch that zeroes its work counter).
    bias [B|1,Hq|1,pps*page] bf16/fp32: additive logit bias per key position."""
    if q.dim() != 3 or k_pages.dim() != 4:
        raise _bad(f"q must be [B,Hq,D] and k_pages [Hkv,P,page,D], got {list(q.shape)}, {list(k_pages.shape)}")
    b, hq, d = q.shape
    hkv, num_pages, page_size, dk = k_pages.shape
    if dk != d:
        raise _bad(f"head_dim of k_pages ({dk}) differs from q's ({d})")
    _want_shape("v_pages", v_pages, k_pages.shape)
    if hkv <= 0 or hq % hkv != 0:
        raise _bad(f"num_q_heads {hq} is not divisible by num_kv_heads {hkv}")
    if page_tables.dim() != 2 or page_tables.shape[0] != b:
        raise _bad(f"page_tables must be [{b}, pages_per_seq], got {list(page_tables.shape)}")
    _want_shape("lengths", lengths, (b,))
    if page_tables.dtype != torch.int32 or lengths.dtype != torch.int32:
        raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, "page_tables and lengths must be int32")
    if k_pages.dtype != q.dtype or v_pages.dtype != q.dtype:
        raise AxlError(_lib.AXL_ERR_UNSUPPORTED, "q and the pools must share one dtype")
    for name, x in (("q", q), ("k_pages", k_pages), ("v_pages", v_pages), ("page_tables", page_tables), ("lengths", lengths)):
        if not x.is_contiguous():
            raise AxlError(_lib.AXL_ERR_UNSUPPORTED, f"{name} must be contiguous")
    _check_decode_out_ws(q, out, workspace)
    if workspace_reused and workspace is None:
        raise _bad("workspace_reused needs the workspace of the earlier call")
    _require_cuda(q, k_pages, v_pages, page_tables, lengths, out, workspace, bias)
    lib = _lib.load()
    if out is None:
        out = torch.empty((b, hq, d), dtype=q.dtype, device=q.device)
    bias_blk, _keep = _decode_bias(bias, b, hq, page_size * page_tables.shape[1])
    p = AxlPagedDecodeParams(
        q=q.data_ptr(), k_pages=k_pages.data_ptr(), v_pages=v_pages.data_ptr(),
        page_tables=page_tables.data_ptr(), lengths=lengths.data_ptr(), out=out.data_ptr(),
        batch=b, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, num_pages=num_pages,
        page_size=page_size, pages_per_seq=page_tables.shape[1],
        dtype=_lib.dtype_code(q.dtype), sliding_window=int(sliding_window),
        softmax_scale=float(softmax_scale), workspace=None, workspace_bytes=0,
        flags=_decode_flags(deterministic, workspace_reused), bias=bias_blk,
    )
    need = int(lib.axl_paged_decode_workspace_bytes(ctypes.byref(p)))
    if workspace is None or workspace.numel() < need:
        if workspace_reused:
            raise AxlError(_lib.AXL_ERR_WORKSPACE, f"workspace needs {need} bytes, got {workspace.numel()}")
        workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=q.device)
    p.workspace = workspace.data_ptr()
    p.workspace_bytes = workspace.numel()
    _lib.check(lib.axl_paged_decode(ctypes.byref(p), _lib.current_stream_ptr()))
    return out


def paged_decode_workspace_bytes(batch: int, num_q_heads: int, num_kv_heads: int, head_dim: int,
                                 pages_per_seq: int, page_size: int = 16, with_bias: bool = False) -> int:
    """Bytes of device workspace `paged_decode` needs for these shapes (bf16)."""
    lib = _lib.load()
    p = AxlPagedDecodeParams(
        batch=batch, num_q_heads=num_q_heads, num_kv_heads=num_kv_heads, head_dim=head_dim,
        num_pages=batch * pages_per_seq, page_size=page_size, pages_per_seq=pages_per_seq,
        dtype=_lib.dtype_code(torch.bfloat16), sliding_window=-1, softmax_scale=1.0,
        bias=AxlDecodeBias(bias=256 if with_bias else None),
    )
    return int(lib.axl_paged_decode_workspace_bytes(ctypes.byref(p)))


def decode(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    lengths: torch.Tensor,
    *,
    softmax_scale: float = 1.0,
    sliding_window: int = -1,
    workspace: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    deterministic: bool = False,
    workspace_reused: bool = False,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """q [B,Hq,D]; k/v [B,S,Hkv,D]; lengths [B] int32 -> [B,Hq,D].  Lengths are clamped to [0, S]; a
    sequence of length 0 yields zeros.  `deterministic` / `workspace_reused`: see `paged_decode`.
    bias [B|1,Hq|1,S] bf16/fp32: additive logit bias per key position."""
    if q.dim() != 3 or k.dim() != 4:
        raise _bad(f"q must be [B,Hq,D] and k [B,S,Hkv,D], got {list(q.shape)}, {list(k.shape)}")
    b, hq, d = q.shape
    s, hkv = k.shape[1], k.shape[2]
    if k.shape[0] != b or k.shape[3] != d:
        raise _bad(f"k {list(k.shape)} does not match q {list(q.shape)} in batch / head_dim")
    _want_shape("v", v, k.shape)
    if hkv <= 0 or hq % hkv != 0:
        raise _bad(f"num_q_heads {hq} is not divisible by num_kv_heads {hkv}")
    _want_shape("lengths", lengths, (b,))
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise AxlError(_lib.AXL_ERR_UNSUPPORTED, "q, k, v must share one dtype")
    if not q.is_contiguous():
        raise AxlError(_lib.AXL_ERR_UNSUPPORTED, "q must be contiguous")
    if lengths.dtype != torch.int32 or not lengths.is_contiguous():
        raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, "lengths must be contiguous int32")
    _check_decode_out_ws(q, out, workspace)
    if workspace_reused and workspace is None:
        raise _bad("workspace_reused needs the workspace of the earlier call")
    _require_cuda(q, k, v, lengths, out, workspace, bias)
    lib = _lib.load()
    if out is None:
        out = torch.empty((b, hq, d), dtype=q.dtype, device=q.device)
    bias_blk, _keep = _decode_bias(bias, b, hq, s)
    p = AxlDecodeParams(
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(), lengths=lengths.data_ptr(),
        out=out.data_ptr(), k_strides=_lib.strides4(k), v_strides=_lib.strides4(v),
        batch=b, kv_len=s, num_q_heads=hq, num_kv_heads=hkv, head_dim=d,
        dtype=_lib.dtype_code(q.dtype), sliding_window=int(sliding_window),
        softmax_scale=float(softmax_scale), workspace=None, workspace_bytes=0,
        flags=_decode_flags(deterministic, workspace_reused), bias=bias_blk,
    )
    need = int(lib.axl_decode_workspace_bytes(ctypes.byref(p)))
    if workspace is None or workspace.numel() < need:
        if workspace_reused:
            raise AxlError(_lib.AXL_ERR_WORKSPACE, f"workspace needs {need} bytes, got {workspace.numel()}")
        workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=q.device)
    p.workspace = workspace.data_ptr()
    p.workspace_bytes = workspace.numel()
    _lib.check(lib.axl_decode(ctypes.byref(p), _lib.current_stream_ptr()))
    return out


def paged_kv_insert(
    k_pages: Optional[torch.Tensor],
    v_pages: Optional[torch.Tensor],
    k_proj: Optional[torch.Tensor],
    v_proj: Optional[torch.Tensor],
    page_indices: torch.Tensor,
    key_positions: torch.Tensor,
) -> None:
    """Writes one new token per sequence into the pools, IN PLACE.

    pools [Hkv,P,page,D]; k_proj/v_proj [B,Hkv,D] (any batch/head strides, dense in D);
    page_indices [B,pps] int32; key_positions [B] int32, or [1] to use one position for all."""
    pool = k_pages if k_pages is not None else v_pages
    proj = k_proj if k_proj is not None else v_proj
    if pool is None or proj is None:
        raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, "nothing to insert")
    _require_cuda(pool, proj, page_indices, key_positions)
    lib = _lib.load()
    if pool.dim() != 4 or page_indices.dim() != 2:
        raise _bad(f"pools must be [Hkv,P,page,D] and page_indices [B,pps], got {list(pool.shape)}, {list(page_indices.shape)}")
    if k_pages is not None and v_pages is not None and tuple(k_pages.shape) != tuple(v_pages.shape):
        raise _bad(f"k_pages {list(k_pages.shape)} and v_pages {list(v_pages.shape)} differ")
    hkv, num_pages, page_size, d = pool.shape
    b = page_indices.shape[0]
    for name, x in (("k_pages", k_pages), ("v_pages", v_pages), ("page_indices", page_indices),
                    ("key_positions", key_positions)):
        if x is not None and not x.is_contiguous():
            raise AxlError(_lib.AXL_ERR_UNSUPPORTED, f"{name} must be contiguous")
    for name, x in (("k_proj", k_proj), ("v_proj", v_proj)):
        if x is not None and (tuple(x.shape) != (b, hkv, d) or x.stride(-1) != 1 or x.dtype != pool.dtype):
            raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, f"{name} must be [B,Hkv,D] of the pool dtype, dense in D")
    if page_indices.dtype != torch.int32 or key_positions.dtype != torch.int32:
        raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, "page_indices and key_positions must be int32")
    if key_positions.numel() not in (1, b):
        raise AxlError(_lib.AXL_ERR_INVALID_ARGUMENT, "key_positions must hold 1 or batch values")
    p = AxlPageInsertParams(
        k_pages=None if k_pages is None else k_pages.data_ptr(),
        v_pages=None if v_pages is None else v_pages.data_ptr(),
        k_proj=None if k_proj is None else k_proj.data_ptr(),
        v_proj=None if v_proj is None else v_proj.data_ptr(),
        page_indices=page_indices.data_ptr(), key_positions=key_positions.data_ptr(),
        k_proj_batch_stride=0 if k_proj is None else k_proj.stride(0),
        k_proj_head_stride=0 if k_proj is None else k_proj.stride(1),
        v_proj_batch_stride=0 if v_proj is None else v_proj.stride(0),
        v_proj_head_stride=0 if v_proj is None else v_proj.stride(1),
        batch=b, num_kv_heads=hkv, head_dim=d, num_pages=num_pages, page_size=page_size,
        pages_per_seq=page_indices.shape[1], dtype=_lib.dtype_code(pool.dtype),
        broadcast_positions=int(key_positions.numel() == 1 and b > 1),
    )
    _lib.check(lib.axl_paged_kv_insert(ctypes.byref(p), _lib.current_stream_ptr()))
