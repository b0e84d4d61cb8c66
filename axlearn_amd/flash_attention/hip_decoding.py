"""Single-token decode kernels (contiguous and paged KV) behind the dispatch API.

`HipDecoding` stands where `GPUDecoding` does (axlearn/common/flash_attention/gpu_decoding.py:
286-352) and `HipPagedAttention` where `GPUPagedAttention` does (gpu_paged_attention.py:299-379).
Both take the decode position from the mask bias: kv length = target_positions[:, -1] + 1
(gpu_decoding.py:314, gpu_paged_attention.py:344).
"""

from __future__ import annotations

from typing import Optional

import torch

from axlearn_amd import ops
from axlearn_amd.attention_bias import (
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
    """-1 for plain causal decoding, w for a sliding window, None if the mask is not structured."""
    kind = classify_mask_bias(mask)
    if kind is None or kind[0] == ops.MASK_NONE:
        return None
    return -1 if kind[0] == ops.MASK_CAUSAL else kind[1]


def _lengths(mask: MaskFnAttentionBias, batch_size: int, device) -> Tensor:
    if mask is None or getattr(mask, "target_positions", None) is None:
        raise ValueError("Cannot retrieve MaskFnAttentionBias or target_positions.")
    lengths = (mask.target_positions[:, -1] + 1).to(device=device, dtype=torch.int32)
    return lengths.expand(batch_size).contiguous()


def _common_checks(self, input_batch: Nested, heads_per_kv: int) -> bool:
    query = input_batch["query"]
    if input_batch.get("logit_sink") is not None:
        return self._log_unsupported("logit_sink is not supported.")
    if query.dtype not in (torch.bfloat16, torch.float16, torch.float32) or input_batch["key"].dtype != query.dtype:
        return self._log_unsupported(
            f"{query.dtype=} / {input_batch['key'].dtype=} (supported: bfloat16, float16 or float32, the same for both)"
        )
    if query.shape[-1] not in (64, 128):
        return self._log_unsupported(f"head_dim {query.shape[-1]} (supported: 64, 128)")
    if heads_per_kv > 16:
        return self._log_unsupported(f"{heads_per_kv} query heads per kv head (supported: <= 16)")
    if not (self.cfg.softmax_scale > 0.0):
        return self._log_unsupported(f"{self.cfg.softmax_scale=} must be positive")
    mask, explicit_bias = split(input_batch["bias"], MaskFnAttentionBias)
    if explicit_bias.has_value():
        return self._log_unsupported("explicit (dense) bias is not supported.")
    if _decode_window(mask) is None:
        return self._log_unsupported("decode needs a causal or sliding-window mask with target_positions.")
    if not query.is_cuda:
        return self._log_unsupported("tensors are not on the GPU.")
    return True


class HipDecoding(BaseSingleStepDecoding):
    """Split-K flash decoding over a contiguous [B,S,Hkv,D] cache."""

    def is_supported(self, input_batch: Nested, kv_cache_type: Optional[type[BaseKVCache]]) -> bool:
        if not super().is_supported(input_batch, kv_cache_type=kv_cache_type):
            return False
        if kv_cache_type != KVCache:
            return self._log_unsupported(f"{kv_cache_type=}")
        return _common_checks(self, input_batch, input_batch["query"].shape[2] // input_batch["key"].shape[2])

    def __call__(self, input_batch: Nested) -> Tensor:
        query, key, value = input_batch["query"], input_batch["key"], input_batch["value"]
        mask, _ = split(input_batch["bias"], MaskFnAttentionBias)
        batch_size, _, q_heads, head_dim = query.shape
        lengths = _lengths(mask, batch_size, query.device)
        out = ops.decode(
            query.reshape(batch_size, q_heads, head_dim), key, value, lengths,
            softmax_scale=float(self.cfg.softmax_scale), sliding_window=_decode_window(mask),
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
        if key.shape[2] != 16:
            return self._log_unsupported(f"page size {key.shape[2]} (supported: 16)")
        if input_batch["page_tables"].dtype != torch.int32:
            return self._log_unsupported("page_tables must be int32")
        return _common_checks(self, input_batch, input_batch["query"].shape[2] // key.shape[0])

    def __call__(self, input_batch: Nested) -> Tensor:
        query, key, value = input_batch["query"], input_batch["key"], input_batch["value"]
        page_tables = input_batch["page_tables"]
        mask, _ = split(input_batch["bias"], MaskFnAttentionBias)
        batch_size, _, q_heads, head_dim = query.shape
        lengths = _lengths(mask, batch_size, query.device)
        out = ops.paged_decode(
            query.reshape(batch_size, q_heads, head_dim), key, value, page_tables.contiguous(), lengths,
            softmax_scale=float(self.cfg.softmax_scale), sliding_window=_decode_window(mask),
        )
        return out.reshape(batch_size, 1, q_heads, head_dim)
