"""JAX side of the XLA FFI binding (csrc/ffi_shim.cc): what an AXLearn maintainer adds next to
axlearn/common/flash_attention/gpu_attention.py to put the HIP kernels behind
`flash_attention_implementation`.

This module needs jax and the FFI library `libaxl_attn_ffi.so` (built from csrc/ffi_shim.cc against
jaxlib's `xla/ffi/api/ffi.h`).  Neither exists in this repository's environment, so the package never
imports it: it is the source of the reference-side binding, kept next to the torch host mirror
(`hip_attention.py`, `hip_decoding.py`) whose behaviour it repeats call for call.  The tests run it under
eager stand-ins for the few jax names it uses (tests/jax_stand_in.py: torch tensors for arrays, and an
`ffi_call` that hands operands, results and attributes to the handlers of csrc/ffi_shim.cc, built against
a stand-in for jaxlib's header), which shows that its classes and its custom_vjp pair give the torch
side's bits with the workspace sizes computed here; XLA, jax's own machinery and the shim against the
real header stay untested.

It mirrors, name for name:
  * `flash_attention` with its `jax.custom_vjp` and residuals `(q, k, v, bias, segment_ids, dropout mask,
    logit_sink, out, lse)` (gpu_attention.py:247-287, :420-424, :789): `out` and `lse` carry
    `checkpoint_name(..., f"gpu_attention.{FLASH_ATTN_RESIDUAL_NAME}")`, the name the remat policy
    `save_and_offload_only_these_names_regex` matches (axlearn/common/flash_attention/remat.py:9-58);
  * `PallasGPUFlashAttention` (gpu_attention.py:929-992) as `HipFlashAttention` (any head_dim up to 128,
    `logit_sink`, and incremental prefill over a contiguous cache, as the torch-side class), `GPUDecoding`
    (gpu_decoding.py:286-352) as `HipDecoding`, `GPUPagedAttention` (gpu_paged_attention.py:299-379)
    as `HipPagedAttention`, to be listed first in `BACKENDS["gpu"]` / `PAGED_ATTN_BACKENDS["gpu"]`
    (flash_attention/utils.py:31-58);
  * `gpu_scatter_update_pages_shmap_fn` (kv_cache/paged_kv_cache_gpu_kernel.py:36-60) as
    `hip_scatter_update_pages`.
"""

# pylint: disable=import-error,too-many-arguments
from __future__ import annotations

import ctypes
import functools
import os

import jax
import jax.numpy as jnp
import numpy as np
from jax.ad_checkpoint import checkpoint_name

from axlearn.common.attention_bias import (  # the reference's own types: this file lives in its tree
    NEG_INF,
    BaseAttentionBias,
    CausalAttentionBias,
    MaskFnAttentionBias,
    SegmentIdAttentionBias,
    SlidingWindowAttentionBias,
    split,
)
from axlearn.common.flash_attention.common import (
    BaseFlashAttention,
    BasePagedAttention,
    BaseSingleStepDecoding,
    repeat_kv_heads,  # noqa: F401  (NOT used: K/V go to the kernels with their own Hkv heads)
)
from axlearn.common.flash_attention.remat import FLASH_ATTN_RESIDUAL_NAME
from axlearn.common.utils import Nested, Tensor

_HERE = os.path.dirname(os.path.abspath(__file__))
_FFI_LIB = ctypes.CDLL(os.path.join(_HERE, "..", "libaxl_attn_ffi.so"))
_CORE_LIB = ctypes.CDLL(os.path.join(_HERE, "..", "libaxl_attn_hip.so"))

if _FFI_LIB.axl_ffi_shim_abi_version() != _CORE_LIB.axl_abi_version():
    raise ImportError(f"libaxl_attn_ffi.so was built against ABI {_FFI_LIB.axl_ffi_shim_abi_version()} of "
                      f"include/axl_attn.h, libaxl_attn_hip.so implements {_CORE_LIB.axl_abi_version()}: rebuild the shim")
for _name in ("AxlFlashFwd", "AxlFlashBwd", "AxlDecode", "AxlPagedDecode", "AxlPagedKvInsert"):
    jax.ffi.register_ffi_target(_name, jax.ffi.pycapsule(getattr(_FFI_LIB, _name)), platform="ROCM")

MASK_NONE, MASK_CAUSAL, MASK_SLIDING_WINDOW = 0, 1, 2
DECODE_DETERMINISTIC = 1


def _empty(dtype) -> Tensor:
    """Stand-in for an absent optional operand (XLA FFI has no optional buffers)."""
    return jnp.zeros((0,), dtype)


def _mask_of(bias: BaseAttentionBias):
    """(mask_kind, window, segment_ids, dense bias or None): the structured parts the kernels evaluate
    arithmetically, as `PallasGPUFlashAttention.__call__` splits them (gpu_attention.py:972-974)."""
    mask, segment_ids, explicit = split(bias, MaskFnAttentionBias, SegmentIdAttentionBias)
    kind, window = MASK_NONE, 0
    if isinstance(mask, SlidingWindowAttentionBias):
        kind, window = MASK_SLIDING_WINDOW, int(mask.sliding_window_size)
    elif isinstance(mask, CausalAttentionBias):
        kind = MASK_CAUSAL
    elif mask.has_value():
        explicit = explicit + mask  # an arbitrary mask_fn: materialised as a bias, once
    seg = segment_ids.segment_ids if segment_ids.has_value() else None
    return kind, window, seg, (explicit.value() if explicit.has_value() else None)


# The backward can keep dS in its workspace where the library has that path (AXL_BWD_DS_WORKSPACE in
# include/axl_attn.h: about T*S bytes per (batch, head) of scratch that XLA allocates for the call, for a
# backward of 5 GEMMs instead of 7).  None: do so whenever that scratch fits BWD_WORKSPACE_LIMIT_BYTES,
# whole or a few kv heads at a time (the same rule as HipFlashAttention.Config.bwd_ds_workspace /
# bwd_workspace_limit_bytes on the torch side, ops.select_ds_slice); True / False force the choice.  The size query below sees the flag that was chosen, so the
# scratch result of the custom call grows with it.
BWD_DS_WORKSPACE = None
BWD_WORKSPACE_LIMIT_BYTES = 18 << 30  # a sixteenth of an MI355X's 288 GB
_AXL_BWD_DS_WORKSPACE = 1


def _bwd_workspace_bytes(b, t, s, hq, hkv, d, dtype_code, mask_kind, has_seg, flags) -> int:
    """axl_flash_bwd_workspace_bytes for these shapes (a host-side size query of the core library)."""
    from axlearn_amd._lib import AxlFlashBwdParams  # the ctypes mirror of include/axl_attn.h

    p = AxlFlashBwdParams(batch=b, q_len=t, kv_len=s, num_q_heads=hq, num_kv_heads=hkv, head_dim=d,
                          dtype=dtype_code, mask_kind=mask_kind, segment_ids=1 if has_seg else None, flags=flags)
    _CORE_LIB.axl_flash_bwd_workspace_bytes.restype = ctypes.c_size_t
    return int(_CORE_LIB.axl_flash_bwd_workspace_bytes(ctypes.byref(p)))


_DTYPE_CODE = {jnp.dtype(jnp.bfloat16): 0, jnp.dtype(jnp.float32): 1, jnp.dtype(jnp.float16): 2}


@functools.partial(jax.custom_vjp, nondiff_argnums=(7, 8, 9, 10))
def flash_attention(query, key, value, bias, segment_ids, dropout_mask, logit_sink, softmax_scale, mask_kind,
                    sliding_window, dropout_rate):
    """Same contract as gpu_attention.py:250-287 with the block-size / warp arguments gone (the kernels
    pick their own tiles), the dropout mask instead of the prng key (drawn by the caller with
    `jax.random.bernoulli(prng_key, dropout_rate, [B,H,T,S])`, as :374-385 does before its kernel), and
    `logit_sink` [Hq] (attention.py:608-626; None for none), which gets a gradient like q, k and v."""
    out, _ = _fwd_call(query, key, value, bias, segment_ids, dropout_mask, logit_sink, softmax_scale, mask_kind,
                       sliding_window, dropout_rate)
    return out


def _fwd_call(query, key, value, bias, segment_ids, dropout_mask, logit_sink, softmax_scale, mask_kind,
              sliding_window, dropout_rate, q_pos_offsets=None):
    b, t, hq, _ = query.shape
    out_type = jax.ShapeDtypeStruct(query.shape, query.dtype)
    lse_type = jax.ShapeDtypeStruct((b, hq, t), jnp.float32)
    return jax.ffi.ffi_call("AxlFlashFwd", (out_type, lse_type))(
        query, key, value,
        _empty(jnp.int32) if segment_ids is None else segment_ids.astype(jnp.int32),
        _empty(jnp.float32) if logit_sink is None else logit_sink.astype(jnp.float32),
        _empty(jnp.float32) if bias is None else bias,
        _empty(jnp.uint8) if dropout_mask is None else dropout_mask.astype(jnp.uint8),
        _empty(jnp.int32) if q_pos_offsets is None else q_pos_offsets.astype(jnp.int32),
        softmax_scale=np.float32(softmax_scale), mask_kind=np.int32(mask_kind),
        sliding_window=np.int32(sliding_window), q_pos_offset=np.int32(0), dropout_rate=np.float32(dropout_rate))


def _flash_fwd(query, key, value, bias, segment_ids, dropout_mask, logit_sink, softmax_scale, mask_kind,
               sliding_window, dropout_rate):
    out, lse = _fwd_call(query, key, value, bias, segment_ids, dropout_mask, logit_sink, softmax_scale, mask_kind,
                         sliding_window, dropout_rate)
    # The names the remat policy looks for (remat.py:13-58): saving or offloading exactly these two
    # tensors lets the backward skip the forward kernel.
    out = checkpoint_name(out, f"gpu_attention.{FLASH_ATTN_RESIDUAL_NAME}")
    lse = checkpoint_name(lse, f"gpu_attention.{FLASH_ATTN_RESIDUAL_NAME}")
    return out, (query, key, value, bias, segment_ids, dropout_mask, logit_sink, out, lse)


def _flash_bwd(softmax_scale, mask_kind, sliding_window, dropout_rate, res, d_out):
    query, key, value, bias, segment_ids, dropout_mask, logit_sink, out, lse = res
    b, t, hq, d = query.shape
    s, hkv = key.shape[1], key.shape[2]
    size_args = (b, t, s, hq, hkv, d, _DTYPE_CODE[jnp.dtype(query.dtype)], mask_kind, segment_ids is not None)
    flags = _AXL_BWD_DS_WORKSPACE if BWD_DS_WORKSPACE or BWD_DS_WORKSPACE is None else 0
    ws_bytes = _bwd_workspace_bytes(*size_args, flags)
    if BWD_DS_WORKSPACE is None and flags and ws_bytes > BWD_WORKSPACE_LIMIT_BYTES:
        # Too large for the automatic choice in one piece: the dS of as many kv heads at a time as fit
        # (AXL_BWD_DS_SLICE_KV_HEADS(n) = n << 8 in the flags; the kernels then run slice after slice),
        # if a slice still gives each of the 256 CUs a dK/dV workgroup; else the recomputing pair.
        per_head = b * (s // 128) // (2 if mask_kind == 1 else 1)   # AXL_MASK_CAUSAL: two key blocks per workgroup
        heads = hkv - 1
        while heads >= 1 and _bwd_workspace_bytes(*size_args, flags | (heads << 8)) > BWD_WORKSPACE_LIMIT_BYTES:
            heads -= 1
        flags = flags | (heads << 8) if heads >= 1 and heads * per_head >= 256 else 0
        ws_bytes = _bwd_workspace_bytes(*size_args, flags)
    dq, dk, dv, d_sink, _ = jax.ffi.ffi_call(
        "AxlFlashBwd",
        (jax.ShapeDtypeStruct(query.shape, query.dtype), jax.ShapeDtypeStruct(key.shape, key.dtype),
         jax.ShapeDtypeStruct(value.shape, value.dtype),
         jax.ShapeDtypeStruct((0,) if logit_sink is None else (hq,), jnp.float32),
         jax.ShapeDtypeStruct((ws_bytes,), jnp.uint8)),
    )(query, key, value, out, d_out, lse,
      _empty(jnp.int32) if segment_ids is None else segment_ids.astype(jnp.int32),
      _empty(jnp.float32) if logit_sink is None else logit_sink.astype(jnp.float32),
      _empty(jnp.float32) if bias is None else bias,
      _empty(jnp.uint8) if dropout_mask is None else dropout_mask.astype(jnp.uint8),
      softmax_scale=np.float32(softmax_scale), mask_kind=np.int32(mask_kind), sliding_window=np.int32(sliding_window),
      q_pos_offset=np.int32(0), dropout_rate=np.float32(dropout_rate), flags=np.int32(flags))
    # No gradient for bias, segment ids or the dropout mask, as `_mha_backward` returns (:786).
    return dq, dk, dv, None, None, None, (None if logit_sink is None else d_sink.astype(logit_sink.dtype))


flash_attention.defvjp(_flash_fwd, _flash_bwd)


def _width(head_dim: int):
    """Compiled width the kernels run a head dim at: 64 or 128 (None above that, gpu_attention.py:954)."""
    return 64 if head_dim <= 64 else (128 if head_dim <= 128 else None)


def _runs_at_native_head_dim(query: Tensor, key: Tensor, aux: bool) -> bool:
    """Head dims 64 and 128 always; other multiples of 8 in bf16 / f16 without bias or dropout mask when
    the (dense) rows are at least one compiled width apart.  Everything else is zero-padded to the width:
    zero columns of q / k add nothing to the logits, zero columns of v give output columns that are
    sliced off again (the Pallas kernel pads inside its blocks instead, gpu_attention.py:172-176)."""
    d = query.shape[-1]
    if d in (64, 128):
        return True
    if d % 8 != 0 or aux or query.dtype == jnp.float32:
        return False
    return query.shape[2] * d >= _width(d) and key.shape[2] * d >= _width(d)


def _pad_last(x: Tensor, width: int) -> Tensor:
    return x if x.shape[-1] == width else jnp.pad(x, ((0, 0),) * (x.ndim - 1) + ((0, width - x.shape[-1]),))


class HipFlashAttention(BaseFlashAttention):
    """Stands where `PallasGPUFlashAttention` does (gpu_attention.py:929-992).  With `kv_cache_type=KVCache`
    and more than one query row it serves incremental prefill (utils_test.py:361-478): a chunk of queries
    per sequence at its own offset into the contiguous cache, forward only."""

    _kv_cache_type = None

    def _incremental_supported(self, input_batch) -> bool:
        query, key = input_batch["query"], input_batch["key"]
        if key.shape[1] % 128 != 0:
            return self._log_unsupported(f"{key.shape[1]=} is not divisible by 128")
        if self.config.dropout_rate != 0.0:
            raise ValueError("Dropout rate cannot be set for decoding!")
        mask, segment_ids, explicit = split(input_batch["bias"], MaskFnAttentionBias, SegmentIdAttentionBias)
        if segment_ids.has_value() or explicit.has_value():
            return self._log_unsupported("incremental prefill takes a causal or sliding-window mask only.")
        if not isinstance(mask, (CausalAttentionBias, SlidingWindowAttentionBias)) or mask.target_positions is None:
            return self._log_unsupported("incremental prefill needs a causal / sliding-window mask with target_positions.")
        if mask.target_positions.shape[1] != query.shape[1]:
            return self._log_unsupported("target_positions do not match the query length.")
        return True

    def is_supported(self, input_batch: Nested[Tensor | BaseAttentionBias], kv_cache_type=None) -> bool:
        if not super().is_supported(input_batch=input_batch, kv_cache_type=kv_cache_type):
            return False
        query, key = input_batch["query"], input_batch["key"]
        if query.dtype not in (jnp.bfloat16, jnp.float16, jnp.float32) or key.dtype != query.dtype:
            return self._log_unsupported(f"{query.dtype=} / {key.dtype=}")
        if kv_cache_type is not None:
            if kv_cache_type.__name__ != "KVCache":
                return self._log_unsupported(f"{kv_cache_type=}")
            if not self._incremental_supported(input_batch):
                return False
        elif not self._check_block_size(input_batch=input_batch, block_size=128):
            return False
        self._kv_cache_type = kv_cache_type
        if _width(query.shape[-1]) is None:
            return self._log_unsupported(f"head_dim {query.shape[-1]} > 128")
        if self.config.dropout_rate > 0.0 and input_batch.get("prng_key", None) is None:
            return self._log_unsupported("dropout needs input_batch['prng_key'].")
        return True

    def _incremental_prefill(self, input_batch) -> Tensor:
        """Queries at per-sequence offsets into the cache; rows padded up to the 128-row block.  The
        positions of a chunk are taken to be consecutive (they are, in `extend_step`)."""
        cfg = self.config
        query, key, value = input_batch["query"], input_batch["key"], input_batch["value"]
        mask, _, _ = split(input_batch["bias"], MaskFnAttentionBias, SegmentIdAttentionBias)
        window = int(mask.sliding_window_size) if isinstance(mask, SlidingWindowAttentionBias) else 0
        b, t, _, d = query.shape
        offsets = jnp.broadcast_to(mask.target_positions[:, 0], (b,)).astype(jnp.int32)
        width = d if _runs_at_native_head_dim(query, key, aux=False) else _width(d)
        rows = -(-t // 128) * 128
        q = jnp.pad(query, ((0, 0), (0, rows - t), (0, 0), (0, width - d)))
        out, _ = _fwd_call(q, _pad_last(key, width), _pad_last(value, width), None, None, None,
                           input_batch.get("logit_sink", None), cfg.softmax_scale,
                           MASK_SLIDING_WINDOW if window else MASK_CAUSAL, window, 0.0, q_pos_offsets=offsets)
        return out[:, :t, :, :d]

    @functools.partial(jax.jit, static_argnames=["self"])
    def __call__(self, input_batch: Nested[Tensor | BaseAttentionBias]) -> Tensor:
        if self._kv_cache_type is not None:
            return self._incremental_prefill(input_batch)
        cfg = self.config
        query, key, value = input_batch["query"], input_batch["key"], input_batch["value"]
        mask_kind, window, segment_ids, dense = _mask_of(input_batch["bias"])
        dropout_mask = None
        if cfg.dropout_rate > 0.0:
            b, t, hq, _ = query.shape
            dropout_mask = jax.random.bernoulli(input_batch["prng_key"], cfg.dropout_rate, (b, hq, t, key.shape[1]))
        d = query.shape[-1]
        if not _runs_at_native_head_dim(query, key, aux=dense is not None or dropout_mask is not None):
            query, key, value = (_pad_last(x, _width(d)) for x in (query, key, value))
        # K / V keep their Hkv heads: no repeat_kv_heads (gpu_attention.py:975-976 repeats them).
        out = flash_attention(query, key, value, dense, segment_ids, dropout_mask, input_batch.get("logit_sink", None),
                              cfg.softmax_scale, mask_kind, window, cfg.dropout_rate)
        return out[..., :d]


def _lengths(bias: BaseAttentionBias, batch: int) -> Tensor:
    mask, _ = split(bias, MaskFnAttentionBias)
    if mask is None or mask.target_positions is None:
        raise ValueError("Cannot retrieve MaskFnAttentionBias or target_positions.")
    return jnp.broadcast_to(mask.target_positions[:, -1] + 1, (batch,)).astype(jnp.int32)  # gpu_decoding.py:314


def _decode_mask_and_bias(bias: BaseAttentionBias, lengths: Tensor, kv_len: int):
    """(sliding window for the kernel or -1, bias [B|1, Hq|1, kv_len] or None).  Causal and sliding-window
    masks are evaluated inside the kernel; any other mask fn is evaluated here as the reference's kernels
    evaluate it, `mask_fn(kv_len - 1, key positions)` per sequence (gpu_decoding.py:110,
    gpu_paged_attention.py:108), and handed over as a row of 0 / NEG_INF beside the explicit bias
    [B|1, Hq|1, 1, S] (gpu_decoding.py:327-336)."""
    mask, explicit = split(bias, MaskFnAttentionBias)
    dense = explicit.value()[:, :, 0] if explicit.has_value() else None
    if isinstance(mask, SlidingWindowAttentionBias):
        return int(mask.sliding_window_size), dense
    if isinstance(mask, CausalAttentionBias) or mask.mask is None:
        return -1, dense
    keep = mask.mask((lengths - 1)[:, None], jnp.arange(kv_len)[None, :])
    row = jnp.where(keep, 0.0, NEG_INF).astype(jnp.float32)[:, None, :]
    return -1, row if dense is None else dense.astype(jnp.float32) + row


def _decode_supported(self, input_batch) -> bool:
    """What the decode kernels take, beyond the base classes' checks (the torch-side classes' gate)."""
    query = input_batch["query"]
    if input_batch.get("logit_sink", None) is not None:
        return self._log_unsupported("logit_sink is not supported.")   # as gpu_decoding.py:299
    ok = (jnp.bfloat16, jnp.float16, jnp.float32)
    if query.dtype not in ok or input_batch["key"].dtype not in ok or input_batch["value"].dtype not in ok:
        return self._log_unsupported(f"{query.dtype=} / {input_batch['key'].dtype=}")
    if query.shape[-1] > 128 or query.shape[-1] % 8 != 0:
        return self._log_unsupported(f"head_dim {query.shape[-1]} (supported: multiples of 8 up to 128)")
    if not self.config.softmax_scale > 0.0:
        return self._log_unsupported(f"{self.config.softmax_scale=} must be positive")
    mask, _ = split(input_batch["bias"], MaskFnAttentionBias)
    if mask is None or getattr(mask, "target_positions", None) is None:
        return self._log_unsupported("decode needs a mask bias with target_positions.")
    return True


class HipDecoding(BaseSingleStepDecoding):
    """Stands where `GPUDecoding` does (gpu_decoding.py:286-352)."""

    def is_supported(self, input_batch: Nested[Tensor | BaseAttentionBias], kv_cache_type=None) -> bool:
        if not super().is_supported(input_batch=input_batch, kv_cache_type=kv_cache_type):
            return False
        if kv_cache_type is None or kv_cache_type.__name__ != "KVCache":
            return self._log_unsupported(f"{kv_cache_type=}")
        return _decode_supported(self, input_batch)

    @functools.partial(jax.jit, static_argnames=["self"])
    def __call__(self, input_batch: Nested[Tensor | BaseAttentionBias]) -> Tensor:
        query, key, value = input_batch["query"], input_batch["key"], input_batch["value"]
        b, _, hq, d = query.shape
        lengths = _lengths(input_batch["bias"], b)
        window, dense = _decode_mask_and_bias(input_batch["bias"], lengths, key.shape[1])
        ws = _decode_workspace_bytes(b, hq, key.shape[2], d, key.shape[1], dense is not None)
        out, _ = jax.ffi.ffi_call(
            "AxlDecode", (jax.ShapeDtypeStruct((b, hq, d), query.dtype), jax.ShapeDtypeStruct((ws,), jnp.uint8)),
        )(query.reshape(b, hq, d), key.astype(query.dtype), value.astype(query.dtype), lengths,
          _empty(jnp.float32) if dense is None else dense,
          softmax_scale=np.float32(self.config.softmax_scale), sliding_window=np.int32(window), flags=np.int32(0))
        return out.reshape(b, 1, hq, d)


class HipPagedAttention(BasePagedAttention):
    """Stands where `GPUPagedAttention` does (gpu_paged_attention.py:299-379)."""

    def is_supported(self, input_batch: Nested[Tensor | BaseAttentionBias], kv_cache_type=None) -> bool:
        if not super().is_supported(input_batch=input_batch, kv_cache_type=kv_cache_type):
            return False
        if not self._check_block_size(input_batch, block_size=self.config.gpu_block_size):
            return False
        page_size = input_batch["key"].shape[2]
        # the reference's gate (gpu_paged_attention.py:313-321): fewer than 16 pages per compute block
        if self.config.gpu_block_size / page_size >= 16:
            return self._log_unsupported(f"pages per compute block must stay below 16, got {page_size=}")
        if page_size < 16 or page_size & (page_size - 1):
            return self._log_unsupported(f"page size {page_size} (supported: 16 times a power of two)")
        return _decode_supported(self, input_batch)

    @functools.partial(jax.jit, static_argnames=["self"])
    def __call__(self, input_batch: Nested[Tensor | BaseAttentionBias]) -> Tensor:
        query, key, value = input_batch["query"], input_batch["key"], input_batch["value"]
        page_tables = input_batch["page_tables"]
        b, _, hq, d = query.shape
        kv_len = page_tables.shape[1] * key.shape[2]
        lengths = _lengths(input_batch["bias"], b)
        window, dense = _decode_mask_and_bias(input_batch["bias"], lengths, kv_len)
        ws = _decode_workspace_bytes(b, hq, key.shape[0], d, kv_len, dense is not None)
        out, _ = jax.ffi.ffi_call(
            "AxlPagedDecode", (jax.ShapeDtypeStruct((b, hq, d), query.dtype), jax.ShapeDtypeStruct((ws,), jnp.uint8)),
        )(query.reshape(b, hq, d), key.astype(query.dtype), value.astype(query.dtype), page_tables.astype(jnp.int32),
          lengths, _empty(jnp.float32) if dense is None else dense,
          softmax_scale=np.float32(self.config.softmax_scale), sliding_window=np.int32(window), flags=np.int32(0))
        return out.reshape(b, 1, hq, d)


def _decode_workspace_bytes(b, hq, hkv, d, kv_len, with_bias) -> int:
    from axlearn_amd._lib import AxlDecodeBias, AxlDecodeParams

    p = AxlDecodeParams(batch=b, kv_len=kv_len, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, dtype=0,
                        bias=AxlDecodeBias(bias=256 if with_bias else None))
    _CORE_LIB.axl_decode_workspace_bytes.restype = ctypes.c_size_t
    return int(_CORE_LIB.axl_decode_workspace_bytes(ctypes.byref(p)))  # same size rule as the paged entry point


def hip_scatter_update_pages(k_pages: Tensor, v_pages: Tensor, k_proj: Tensor, v_proj: Tensor,
                             page_indices: Tensor, key_positions: Tensor):
    """`gpu_scatter_update_pages_shmap_fn` (paged_kv_cache_gpu_kernel.py:36-60) for the K and the V pool
    in one call; pools [Hkv,P,page,D], projections [Hkv,B,1,D].  The pools are donated and updated in
    place (`input_output_aliases`, as :57).  Returns the updated (k_pages, v_pages)."""
    return jax.ffi.ffi_call(
        "AxlPagedKvInsert",
        (jax.ShapeDtypeStruct(k_pages.shape, k_pages.dtype), jax.ShapeDtypeStruct(v_pages.shape, v_pages.dtype)),
        input_output_aliases={0: 0, 1: 1},
    )(k_pages, v_pages, k_proj, v_proj, page_indices.astype(jnp.int32), key_positions.reshape(-1).astype(jnp.int32))
