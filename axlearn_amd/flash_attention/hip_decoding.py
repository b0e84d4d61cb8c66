"""Single-token decode kernels (contiguous and paged KV) behind the dispatch API.

`HipDecoding` stands where `GPUDecoding` does (axlearn/common/flash_attention/gpu_decoding.py:
286-352) and `HipPagedAttention` where `GPUPagedAttention` does (gpu_paged_attention.py:299-379).
Both take the decode position from the mask bias: kv length = target_positions[:, -1] + 1
(gpu_decoding.py:314, gpu_paged_attention.py:344).  As in the reference,
  * an explicit bias `[B|1, Hq|1, 1, S]` is added to the scaled logits (gpu_decoding.py:327-336,
    gpu_paged_attention.py:346-348);
  * any `mask_fn` is honoured (gpu_decoding.py:110, gpu_paged_attention.py:108): causal and
    sliding-window masks in closed form inside the kernel, any other as the per-key row
    `mask_fn(length - 1, key positions)` evaluated once on the host and handed over as a 0 / -1e15
    bias row per sequence;
  * K/V of a dtype other than the query's are cast to the query's (gpu_decoding.py:115,133) - here
    ahead of the call, a pass over the cache that same-dtype callers do not pay;
  * any number of query heads per kv head, any head_dim that is a multiple of 8 up to 128.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from axlearn_amd import ops
from axlearn_amd.attention_bias import (
    NEG_INF,
    BaseAttentionBias,
    MaskFnAttentionBias,
    split,
)
from axlearn_amd.flash_attention.common import (
    BasePagedAttention,
    BaseSingleStepDecoding,
    Nested,
    Tensor,
)
from axlearn_amd.flash_attention.hip_attention import classify_mask_bias
from axlearn_amd.kv_cache import BaseKVCache, KVCache


def _decode_window(mask: BaseAttentionBias) -> Optional[int]:
    """-1 for plain causal decoding, w for a sliding window, None if the mask has no closed form in
    the kernel (no mask at all counts as such: every key below the length is visible, which is what
    the causal form gives for the one query at position length - 1)."""
    kind = classify_mask_bias(mask)
    if kind is None:
        return None
    if kind[0] == ops.MASK_NONE:
        return -1
    return -1 if kind[0] == ops.MASK_CAUSAL else kind[1]


def _lengths(mask: MaskFnAttentionBias, batch_size: int, device) -> Tensor:
    if mask is None or getattr(mask, "target_positions", None) is None:
        raise ValueError("Cannot retrieve MaskFnAttentionBias or target_positions.")
    lengths = (mask.target_positions[:, -1] + 1).to(device=device, dtype=torch.int32)
    return lengths.expand(batch_size).contiguous()


def _mask_and_bias(input_batch: Nested, lengths: Tensor, kv_len: int) -> Tuple[int, Optional[Tensor]]:
    """(sliding window for the kernel or -1, bias `[B|1, Hq|1, kv_len]` or None) of a decode call."""
    mask, explicit_bias = split(input_batch["bias"], MaskFnAttentionBias)
    query = input_batch["query"]
    bias = None
    if explicit_bias.has_value():
        value = explicit_bias.value().to(query.device)  # [B|1, Hq|1, 1, S]
        if value.dim() != 4 or value.shape[2] != 1 or value.shape[3] != kv_len:
            raise ValueError(f"Expected a decode bias of shape [B|1, Hq|1, 1, {kv_len}], got {tuple(value.shape)}.")
        bias = value[:, :, 0]
    window = _decode_window(mask)
    if window is None:
        # mask_fn(kv_len - 1, indices), per sequence (gpu_decoding.py:110): a row of 0 / NEG_INF.
        qpos = (lengths.to(torch.int64) - 1)[:, None]
        kpos = torch.arange(kv_len, device=query.device)[None, :]
        keep = torch.as_tensor(mask.mask(qpos, kpos), device=query.device).expand(lengths.shape[0], kv_len)
        row = torch.where(keep, 0.0, NEG_INF).to(torch.float32)[:, None, :]
        bias = row if bias is None else bias.to(torch.float32) + row
        window = -1
    return window, bias


def _common_checks(self, input_batch: Nested) -> bool:
    query = input_batch["query"]
    if input_batch.get("logit_sink") is not None:
        return self._log_unsupported("logit_sink is not supported.")
    ok = (torch.bfloat16, torch.float16, torch.float32)
    if query.dtype not in ok or input_batch["key"].dtype not in ok or input_batch["value"].dtype not in ok:
        return self._log_unsupported(
            f"{query.dtype=} / {input_batch['key'].dtype=} (supported: bfloat16, float16 or float32)"
        )
    if query.shape[-1] > 128 or query.shape[-1] % 8 != 0:
        return self._log_unsupported(f"head_dim {query.shape[-1]} (supported: multiples of 8 up to 128)")
    if not (self.cfg.softmax_scale > 0.0):
        return self._log_unsupported(f"{self.cfg.softmax_scale=} must be positive")
    mask, _ = split(input_batch["bias"], MaskFnAttentionBias)
    if getattr(mask, "target_positions", None) is None:
        return self._log_unsupported("decode needs a mask bias with target_positions.")
    if not query.is_cuda:
        return self._log_unsupported("tensors are not on the GPU.")
    return True


def _as_query_dtype(x: Tensor, query: Tensor) -> Tensor:
    """K/V in the query's dtype (the reference casts each block after loading it)."""
    return x if x.dtype == query.dtype else x.to(query.dtype)


class HipDecoding(BaseSingleStepDecoding):
    """Split-K flash decoding over a contiguous [B,S,Hkv,D] cache."""

    def is_supported(self, input_batch: Nested, kv_cache_type: Optional[type[BaseKVCache]]) -> bool:
        if not super().is_supported(input_batch, kv_cache_type=kv_cache_type):
            return False
        if kv_cache_type != KVCache:
            return self._log_unsupported(f"{kv_cache_type=}")
        return _common_checks(self, input_batch)

    def __call__(self, input_batch: Nested) -> Tensor:
        query, key, value = input_batch["query"], input_batch["key"], input_batch["value"]
        mask, _ = split(input_batch["bias"], MaskFnAttentionBias)
        batch_size, _, q_heads, head_dim = query.shape
        lengths = _lengths(mask, batch_size, query.device)
        window, bias = _mask_and_bias(input_batch, lengths, key.shape[1])
        out = ops.decode(
            query.reshape(batch_size, q_heads, head_dim), _as_query_dtype(key, query), _as_query_dtype(value, query),
            lengths, softmax_scale=float(self.cfg.softmax_scale), sliding_window=window, bias=bias,
        )
        return out.reshape(batch_size, 1, q_heads, head_dim)


class HipPagedAttention(BasePagedAttention):
    """Split-K decode over a paged KV pool [Hkv, pages, page_size, D] with per-sequence page tables."""

    def is_supported(self, input_batch: Nested, kv_cache_type: Optional[type[BaseKVCache]]) -> bool:
        if not super().is_supported(input_batch, kv_cache_type=kv_cache_type):
            return False
        key = input_batch["key"]
        if not self._check_block_size(input_batch, block_size=self.cfg.gpu_block_size):
            return False
        page_size = key.shape[2]
        # the reference's gate (gpu_paged_attention.py:313-321): fewer than 16 pages per compute block
        if self.cfg.gpu_block_size / page_size >= 16:
            return self._log_unsupported(
                f"pages per compute block must stay below 16, got {self.cfg.gpu_block_size} / {page_size}")
        if page_size < 16 or page_size & (page_size - 1):
            return self._log_unsupported(f"page size {page_size} (supported: 16 times a power of two)")
        if input_batch["page_tables"].dtype != torch.int32:
            return self._log_unsupported("page_tables must be int32")
        return _common_checks(self, input_batch)

    def __call__(self, input_batch: Nested) -> Tensor:
        query, key, value = input_batch["query"], input_batch["key"], input_batch["value"]
        page_tables = input_batch["page_tables"]
        mask, _ = split(input_batch["bias"], MaskFnAttentionBias)
        batch_size, _, q_heads, head_dim = query.shape
        lengths = _lengths(mask, batch_size, query.device)
        window, bias = _mask_and_bias(input_batch, lengths, key.shape[2] * page_tables.shape[1])
        out = ops.paged_decode(
            query.reshape(batch_size, q_heads, head_dim), _as_query_dtype(key, query), _as_query_dtype(value, query),
            page_tables.contiguous(), lengths, softmax_scale=float(self.cfg.softmax_scale), sliding_window=window,
            bias=bias,
        )
        return out.reshape(batch_size, 1, q_heads, head_dim)
