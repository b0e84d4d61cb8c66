"""Kernel-class interface and trace-time helpers shared by the HIP attention kernels.

Mirrors the interface part of axlearn/common/flash_attention/common.py: `BaseFlashAttention`
(:144-319), `BaseSingleStepDecoding` (:322-340), `BasePagedAttention` (:343-454), the block-map
helpers (:33-141), `get_segment_ids` (:457-472) and `repeat_kv_heads` (:475-484).  Error behaviour
is the reference's: shapes that make no sense raise `ValueError`; legal-but-unsupported requests log
a reason and return False so that the dispatch falls through to the next candidate.
"""

from __future__ import annotations

import logging
from typing import Any, NamedTuple, Optional

import numpy as np
import torch

from axlearn_amd.attention_bias import BaseAttentionBias, MaskFn, SegmentIdAttentionBias
from axlearn_amd.config import Configurable, config_class
from axlearn_amd.flash_attention.attention_types import FlashAttentionWithShardMapSpecs
from axlearn_amd.kv_cache import BaseKVCache, KVCache, PagedKVCache

Tensor = torch.Tensor
Nested = dict


def validate_contains_paths(tree: dict, paths) -> None:
    for p in paths:
        if p not in tree or tree[p] is None:
            raise ValueError(f"Input is expected to contain '{p}'; instead, it contains: {sorted(tree)}.")


# ------------------------------------------------------------------------------- block maps


def build_mask(
    mask_fn: MaskFn, *, q_seq_len: int, kv_seq_len: int, block_q: int, block_k: int
) -> np.ndarray:
    """[num_q_blocks, num_kv_blocks] bool: True where the tile keeps at least one element
    (common.py:33-80).  Evaluated one tile ROW at a time on whole index vectors, so a 256x256 block
    map costs 256 mask evaluations rather than 65 536."""
    nq = -(-q_seq_len // block_q)
    nk = -(-kv_seq_len // block_k)
    out = np.zeros((nq, nk), dtype=np.bool_)
    cols = torch.arange(nk * block_k, dtype=torch.int32)
    for i in range(nq):
        rows = torch.arange(i * block_q, (i + 1) * block_q, dtype=torch.int32)
        keep = torch.as_tensor(mask_fn(rows[:, None], cols[None, :]))
        out[i] = keep.reshape(block_q, nk, block_k).any(dim=2).any(dim=0).numpy()
    return out


def build_sliding_window_mask(
    *, q_seq_len: int, kv_seq_len: int, block_q: int, block_k: int, sliding_window_size: int
) -> np.ndarray:
    """Closed form of `build_mask(sliding_window_causal_mask(w))` (common.py:83-104): tile (i, j)
    is live iff its first key is not after its last query (causal) and its last key is within the
    window of its first query."""
    nq = -(-q_seq_len // block_q)
    nk = -(-kv_seq_len // block_k)
    q_first = np.arange(nq)[:, None] * block_q
    q_last = q_first + block_q - 1
    k_first = np.arange(nk)[None, :] * block_k
    k_last = k_first + block_k - 1
    return (k_first <= q_last) & (q_first - k_last <= sliding_window_size)


class KVOffsetInfo(NamedTuple):
    """Compacted list of live kv blocks per query block (common.py:107-119)."""

    kv_block_offset: np.ndarray
    kv_block_offset_size: np.ndarray


def query_iterator_indices(block_mask_map: np.ndarray, *, padding: int = 0) -> KVOffsetInfo:
    """common.py:122-141."""
    nq, nk = block_mask_map.shape
    offset = np.full((nq, nk), padding, dtype=np.int32)
    size = block_mask_map.sum(axis=1).astype(np.int32)
    for i in range(nq):
        live = np.nonzero(block_mask_map[i])[0]
        offset[i, : len(live)] = live
    return KVOffsetInfo(kv_block_offset=offset, kv_block_offset_size=size)


def key_value_iterator_indices(block_mask_map: np.ndarray):
    """Column-major counterpart used by the dK/dV pass (gpu_attention.py:91-111)."""
    info = query_iterator_indices(np.ascontiguousarray(block_mask_map.T), padding=0)
    return info.kv_block_offset, info.kv_block_offset_size


# ------------------------------------------------------------------------------- kernel classes


class BaseFlashAttention(Configurable):
    """Common interface of the attention kernels (common.py:144-319)."""

    @config_class
    class Config(Configurable.Config):
        softmax_scale: float = 1.0
        dropout_rate: float = 0.0
        interpret: bool = False
        tpu_block_size: int = 512
        gpu_block_size: int = 128
        backend_overrides: Optional[dict] = None

    def __init__(self, cfg: "BaseFlashAttention.Config"):
        super().__init__(cfg)
        self.cfg = cfg

    def get_backend_overrides(self, name: str, default: Any) -> Any:
        return (self.cfg.backend_overrides or {}).get(name, default)

    def name(self) -> str:
        return self.__class__.__name__

    def _log_unsupported(self, reason: str) -> bool:
        logging.warning("Not using %s because %s", self.name(), reason)
        return False

    def __call__(self, input_batch: Nested) -> Tensor:
        """input_batch: query [B,T,Hq,D], key/value [B,S,Hkv,D], bias: BaseAttentionBias, optional
        prng_key / logit_sink / page_tables.  Returns the context [B,T,Hq,D]."""
        raise NotImplementedError()

    def _validate_input_batch(self, input_batch: Nested) -> None:
        validate_contains_paths(input_batch, paths=["query", "key", "value", "bias"])
        key, value = input_batch["key"], input_batch["value"]
        if key.shape != value.shape:
            raise ValueError(f"Expects {key.shape=} to be equal to {value.shape=}")

    def is_supported(self, input_batch: Nested, kv_cache_type: Optional[type[BaseKVCache]]) -> bool:
        del kv_cache_type
        self._validate_input_batch(input_batch)
        query, key = input_batch["query"], input_batch["key"]
        logit_sink = input_batch.get("logit_sink", None)
        if query.shape[0] != key.shape[0]:
            raise ValueError(
                f"Expects query batch size {query.shape[0]} to be equal to key batch size "
                f"{key.shape[0]}"
            )
        if query.shape[-1] != key.shape[-1]:
            raise ValueError(
                f"Expects query head dim {query.shape[-1]} to be equal to key head dim "
                f"{key.shape[-1]}"
            )
        if query.shape[2] % key.shape[2] != 0:
            raise ValueError(
                f"Expects query num heads {query.shape[2]} to be divisible by num key heads "
                f"{key.shape[2]}"
            )
        if logit_sink is not None and logit_sink.shape[0] != query.shape[2]:
            raise ValueError(
                f"Expects logit sink num heads {logit_sink.shape[0]} to be equal to "
                f"num query heads {query.shape[2]}."
            )
        return True

    def _check_block_size(self, input_batch: Nested, *, block_size: int) -> bool:
        self._validate_input_batch(input_batch)
        q_seq_len = input_batch["query"].shape[1]
        k_seq_len = input_batch["key"].shape[1]
        if q_seq_len % block_size != 0 or k_seq_len % block_size != 0:
            self._log_unsupported(f"{q_seq_len=} or {k_seq_len=} is not divisible by {block_size=}")
            return False
        return True

    def build(self, input_batch: Nested) -> FlashAttentionWithShardMapSpecs:
        del input_batch
        return FlashAttentionWithShardMapSpecs(fn=self)


class BaseSingleStepDecoding(BaseFlashAttention):
    """Checks shared by the single-token decode kernels (common.py:322-340)."""

    def is_supported(self, input_batch: Nested, kv_cache_type: Optional[type[BaseKVCache]]) -> bool:
        if not super().is_supported(input_batch, kv_cache_type=kv_cache_type):
            return False
        if kv_cache_type not in (KVCache, PagedKVCache):
            return self._log_unsupported(f"{kv_cache_type=}")
        if input_batch["query"].shape[1] != 1:
            return self._log_unsupported(f"{input_batch['query'].shape[1]=} != 1")
        if self.cfg.dropout_rate != 0.0:
            raise ValueError("Dropout rate cannot be set for decoding!")
        return True


class BasePagedAttention(BaseSingleStepDecoding):
    """Base of the paged-attention kernels (common.py:343-454).

    input_batch: query [B,1,Hq,D]; key/value page pools [Hkv, total_pages, page_size, D];
    page_tables [B, pages_per_sequence] int32 mapping (sequence, logical page) -> physical page.
    """

    @config_class
    class Config(BaseSingleStepDecoding.Config):
        sparse_ratio: float = 0.8

    def _validate_input_batch(self, input_batch: Nested) -> None:
        super()._validate_input_batch(input_batch)
        validate_contains_paths(input_batch, paths=["page_tables"])

    def _check_block_size(self, input_batch: Nested, block_size: int) -> bool:
        self._validate_input_batch(input_batch)
        page_size = input_batch["key"].shape[2]
        if block_size % page_size != 0:
            self._log_unsupported(f"{block_size=} is not divisible by page size {page_size}")
            return False
        return True

    def is_supported(self, input_batch: Nested, kv_cache_type: Optional[type[BaseKVCache]]) -> bool:
        self._validate_input_batch(input_batch)
        if kv_cache_type != PagedKVCache:
            return self._log_unsupported(f"{kv_cache_type=}")
        query, key = input_batch["query"], input_batch["key"]
        page_tables = input_batch["page_tables"]
        if query.shape[1] != 1:
            return self._log_unsupported(f"{query.shape[1]=} != 1")
        if self.cfg.dropout_rate != 0.0:
            raise ValueError("Dropout rate cannot be set for decoding!")
        logit_sink = input_batch.get("logit_sink", None)
        if logit_sink is not None and logit_sink.shape[0] != query.shape[2]:
            raise ValueError(
                f"Expects logit sink num heads {logit_sink.shape[0]} to be equal to "
                f"num query heads {query.shape[2]}."
            )
        if query.shape[2] % key.shape[0] != 0:
            return self._log_unsupported(
                f"Number of Q heads {query.shape[2]} must be divisible by number of kv heads {key.shape[0]}"
            )
        if query.shape[-1] != key.shape[-1]:
            return self._log_unsupported(
                f"head_dim of Q {query.shape[-1]} must be the same as that of K/V {key.shape[-1]}"
            )
        if page_tables.shape[0] != query.shape[0]:
            return self._log_unsupported(
                "page tables must have the same batch size with query, "
                f"got {page_tables.shape[0]} and {query.shape[0]}"
            )
        return True


def get_segment_ids(*, query: Tensor, key: Tensor, segment_ids: SegmentIdAttentionBias) -> Optional[Tensor]:
    """The [batch, seq] id tensor of a segment bias, or None (common.py:457-472)."""
    if not segment_ids.has_value():
        return None
    if query.shape[1] != key.shape[1]:
        raise ValueError("segment_ids is only supported for query and key with identical lengths.")
    if segment_ids.eval_shape()[0] != query.shape[0]:
        raise ValueError(
            f"segment_ids must have matching batch dim: {segment_ids.eval_shape()} vs. {query.shape[0]}"
        )
    return segment_ids.segment_ids


def repeat_kv_heads(num_q_heads: int, key_or_value: Tensor) -> Tensor:
    """[B,S,Hkv,D] -> [B,S,Hq,D] by repeating each kv head Hq/Hkv times (common.py:475-484).

    The HIP kernels index the shared kv head directly and never call this; it exists for callers
    and tests that want the reference's materialised layout."""
    reps = num_q_heads // key_or_value.shape[-2]
    if reps == 1:
        return key_or_value
    return torch.repeat_interleave(key_or_value, reps, dim=-2)
