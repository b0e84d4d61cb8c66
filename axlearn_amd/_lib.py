"""ctypes binding of libaxl_attn_hip.so (the C ABI declared in include/axl_attn.h).

The library is the only compute path: if it cannot be loaded every kernel entry raises. There is no
PyTorch or CPU fallback anywhere in this package.
"""

from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libaxl_attn_hip.so")

AXL_BF16, AXL_F32, AXL_F16 = 0, 1, 2
MASK_NONE, MASK_CAUSAL, MASK_SLIDING_WINDOW = 0, 1, 2
DECODE_DETERMINISTIC, DECODE_WORKSPACE_REUSED = 1, 2  # AXL_DECODE_* flags
BWD_DS_WORKSPACE = 1  # AXL_BWD_DS_WORKSPACE
AXL_OK, AXL_ERR_INVALID_ARGUMENT, AXL_ERR_UNSUPPORTED, AXL_ERR_WORKSPACE, AXL_ERR_LAUNCH = 0, -1, -2, -3, -4


ABI_VERSION = 7  # AXL_ATTN_ABI_VERSION of include/axl_attn.h these structures mirror


class AxlError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, code: int, message: str):
        super().__init__(f"[axl status {code}] {message}")
        self.code = code


class AxlStrides(ctypes.Structure):
    _fields_ = [("batch", ctypes.c_int64), ("seq", ctypes.c_int64), ("head", ctypes.c_int64)]


class AxlAttnAux(ctypes.Structure):
    _fields_ = [
        ("bias", ctypes.c_void_p),
        ("bias_batch_stride", ctypes.c_int64), ("bias_head_stride", ctypes.c_int64),
        ("bias_row_stride", ctypes.c_int64),
        ("bias_dtype", ctypes.c_int32), ("dropout_rate", ctypes.c_float),
        ("dropout_mask", ctypes.c_void_p),
        ("drop_batch_stride", ctypes.c_int64), ("drop_head_stride", ctypes.c_int64),
        ("drop_row_stride", ctypes.c_int64),
    ]


class AxlFlashFwdParams(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("out", ctypes.c_void_p), ("lse", ctypes.c_void_p), ("segment_ids", ctypes.c_void_p),
        ("q_strides", AxlStrides), ("k_strides", AxlStrides), ("v_strides", AxlStrides),
        ("out_strides", AxlStrides),
        ("batch", ctypes.c_int32), ("q_len", ctypes.c_int32), ("kv_len", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32), ("num_kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("dtype", ctypes.c_int32), ("mask_kind", ctypes.c_int32),
        ("sliding_window", ctypes.c_int32), ("q_pos_offset", ctypes.c_int32),
        ("softmax_scale", ctypes.c_float),
        ("logit_sink", ctypes.c_void_p),
        ("aux", AxlAttnAux),
        ("q_pos_offsets", ctypes.c_void_p),
    ]


class AxlFlashBwdParams(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("out", ctypes.c_void_p), ("d_out", ctypes.c_void_p), ("lse", ctypes.c_void_p),
        ("dq", ctypes.c_void_p), ("dk", ctypes.c_void_p), ("dv", ctypes.c_void_p),
        ("segment_ids", ctypes.c_void_p),
        ("q_strides", AxlStrides), ("k_strides", AxlStrides), ("v_strides", AxlStrides),
        ("out_strides", AxlStrides), ("d_out_strides", AxlStrides),
        ("dq_strides", AxlStrides), ("dk_strides", AxlStrides), ("dv_strides", AxlStrides),
        ("batch", ctypes.c_int32), ("q_len", ctypes.c_int32), ("kv_len", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32), ("num_kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("dtype", ctypes.c_int32), ("mask_kind", ctypes.c_int32),
        ("sliding_window", ctypes.c_int32), ("q_pos_offset", ctypes.c_int32),
        ("softmax_scale", ctypes.c_float),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("logit_sink", ctypes.c_void_p), ("d_logit_sink", ctypes.c_void_p),
        ("aux", AxlAttnAux),
        ("flags", ctypes.c_int32),
    ]


class AxlDecodeBias(ctypes.Structure):
    _fields_ = [
        ("bias", ctypes.c_void_p), ("batch_stride", ctypes.c_int64), ("head_stride", ctypes.c_int64),
        ("dtype", ctypes.c_int32),
    ]


class AxlPagedDecodeParams(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p), ("k_pages", ctypes.c_void_p), ("v_pages", ctypes.c_void_p),
        ("page_tables", ctypes.c_void_p), ("lengths", ctypes.c_void_p), ("out", ctypes.c_void_p),
        ("batch", ctypes.c_int32), ("num_q_heads", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32), ("head_dim", ctypes.c_int32),
        ("num_pages", ctypes.c_int32), ("page_size", ctypes.c_int32),
        ("pages_per_seq", ctypes.c_int32),
        ("dtype", ctypes.c_int32), ("sliding_window", ctypes.c_int32),
        ("softmax_scale", ctypes.c_float),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("flags", ctypes.c_int32),
        ("bias", AxlDecodeBias),
    ]


class AxlDecodeParams(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("lengths", ctypes.c_void_p), ("out", ctypes.c_void_p),
        ("k_strides", AxlStrides), ("v_strides", AxlStrides),
        ("batch", ctypes.c_int32), ("kv_len", ctypes.c_int32), ("num_q_heads", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32), ("head_dim", ctypes.c_int32),
        ("dtype", ctypes.c_int32), ("sliding_window", ctypes.c_int32),
        ("softmax_scale", ctypes.c_float),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("flags", ctypes.c_int32),
        ("bias", AxlDecodeBias),
    ]


class AxlPageInsertParams(ctypes.Structure):
    _fields_ = [
        ("k_pages", ctypes.c_void_p), ("v_pages", ctypes.c_void_p),
        ("k_proj", ctypes.c_void_p), ("v_proj", ctypes.c_void_p),
        ("page_indices", ctypes.c_void_p), ("key_positions", ctypes.c_void_p),
        ("k_proj_batch_stride", ctypes.c_int64), ("k_proj_head_stride", ctypes.c_int64),
        ("v_proj_batch_stride", ctypes.c_int64), ("v_proj_head_stride", ctypes.c_int64),
        ("batch", ctypes.c_int32), ("num_kv_heads", ctypes.c_int32), ("head_dim", ctypes.c_int32),
        ("num_pages", ctypes.c_int32), ("page_size", ctypes.c_int32), ("pages_per_seq", ctypes.c_int32),
        ("dtype", ctypes.c_int32), ("broadcast_positions", ctypes.c_int32),
    ]


EXPORTED_SYMBOLS = (
    "axl_flash_fwd",
    "axl_flash_bwd",
    "axl_flash_bwd_phases",
    "axl_flash_bwd_workspace_bytes",
    "axl_paged_decode",
    "axl_paged_decode_workspace_bytes",
    "axl_paged_decode_static",
    "axl_decode",
    "axl_decode_workspace_bytes",
    "axl_paged_kv_insert",
    "axl_last_error",
    "axl_abi_version",
)

_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """Loads the HIP library, or raises: there is nothing to fall back to."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing. Build it with `make -C axlearn_amd/csrc` (needs hipcc); "
            "axlearn_amd has no non-HIP execution path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    lib.axl_last_error.restype = ctypes.c_char_p
    lib.axl_abi_version.restype = ctypes.c_int
    if lib.axl_abi_version() != ABI_VERSION:
        raise RuntimeError(
            f"{LIB_PATH} has ABI version {lib.axl_abi_version()}, this binding expects {ABI_VERSION}: "
            "rebuild it with `make -C axlearn_amd/csrc`."
        )
    for name, ptype in (
        ("axl_flash_fwd", AxlFlashFwdParams),
        ("axl_flash_bwd", AxlFlashBwdParams),
        ("axl_paged_decode", AxlPagedDecodeParams),
        ("axl_paged_decode_static", AxlPagedDecodeParams),
        ("axl_decode", AxlDecodeParams),
        ("axl_paged_kv_insert", AxlPageInsertParams),
    ):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.POINTER(ptype), ctypes.c_void_p]
    lib.axl_flash_bwd_phases.restype = ctypes.c_int
    lib.axl_flash_bwd_phases.argtypes = [ctypes.POINTER(AxlFlashBwdParams), ctypes.c_int, ctypes.c_void_p]
    for name, ptype in (
        ("axl_flash_bwd_workspace_bytes", AxlFlashBwdParams),
        ("axl_paged_decode_workspace_bytes", AxlPagedDecodeParams),
        ("axl_decode_workspace_bytes", AxlDecodeParams),
    ):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_size_t
        fn.argtypes = [ctypes.POINTER(ptype)]
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != AXL_OK:
        raise AxlError(rc, load().axl_last_error().decode())


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return AXL_BF16
    if dtype == torch.float32:
        return AXL_F32
    if dtype == torch.float16:
        return AXL_F16
    raise AxlError(AXL_ERR_UNSUPPORTED, f"dtype {dtype} (supported: bfloat16, float16, float32)")


def strides4(t: torch.Tensor) -> AxlStrides:
    """Strides of a [batch, seq, heads, head_dim] tensor; the last dim must be dense."""
    if t.dim() != 4 or t.stride(3) != 1:
        raise AxlError(AXL_ERR_UNSUPPORTED, f"expected a 4-d tensor dense in head_dim, got strides {t.stride()}")
    return AxlStrides(t.stride(0), t.stride(1), t.stride(2))


def current_stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()
