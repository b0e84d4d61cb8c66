"""KV-cache marker types and the paged-KV helpers that sit either side of the decode kernels.

`flash_attention_implementation` dispatches on the TYPE of the KV cache
(axlearn/common/flash_attention/utils.py:134; common.py:333, :385); only the types and the page
layout contract are needed here, not the cache layers themselves.
"""

from __future__ import annotations


class BaseKVCache:
    """Stands for axlearn/common/kv_cache/base_kv_cache.py:33 `BaseKVCache`."""


class KVCache(BaseKVCache):
    """Contiguous cache: key/value handed to attention as [batch, kv_len, num_kv_heads, head_dim]
    (axlearn/common/kv_cache/kv_cache.py:20)."""


class PagedKVCache(KVCache):
    """Paged cache: key/value pools [num_kv_heads, total_pages, page_size, head_dim] plus
    page_indices [batch, pages_per_sequence] (axlearn/common/kv_cache/paged_kv_cache.py:106)."""

    # Page id 0 is the padding page and is never written (paged_kv_cache.py:120).
    PADDING_PAGE_ID = 0
