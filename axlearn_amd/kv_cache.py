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


def scatter_update_pages_kernel(*, kv_pages, kv_proj, page_indices, key_positions):
    """Writes the new token of every sequence into `kv_pages`, in place, and returns `kv_pages`.

    Same arguments as the reference's `scatter_update_pages_kernel`
    (axlearn/common/kv_cache/paged_kv_cache.py:62-103) once its `shmap_fn` is bound to the GPU kernel
    (paged_kv_cache_gpu_kernel.py:36-60): kv_pages [num_heads, num_pages, page_size, head_dim];
    kv_proj [num_heads, batch, 1, head_dim]; page_indices [batch, pages_per_batch] int32;
    key_positions [batch, 1] int32.  The reference returns a new array aliased onto the input
    (`input_output_aliases`); here the update is in place.  Page 0 is never written."""
    from axlearn_amd import ops

    if kv_proj.dim() != 4 or kv_proj.shape[2] != 1:
        raise ValueError(f"{kv_proj.shape=}: expected [num_heads, batch, 1, head_dim] (single time step)")
    if key_positions.dim() != 2 or key_positions.shape[1] != 1:
        raise ValueError(f"{key_positions.shape=}: expected [batch, 1]")
    proj = kv_proj[:, :, 0].transpose(0, 1)  # [batch, heads, head_dim] view, no copy
    ops.paged_kv_insert(kv_pages, None, proj, None, page_indices, key_positions.reshape(-1).contiguous())
    return kv_pages


def paged_extend_step(k_pages, v_pages, page_indices, *, k_proj, v_proj, key_positions):
    """The pool update of `PagedKVCache.extend_step` (paged_kv_cache.py:183-240) for one decode step:
    k_proj, v_proj [batch, 1, num_heads, head_dim] are cast to the pool dtype and written at
    key_positions [batch or 1, 1]; both pools are updated by one kernel launch, in place."""
    from axlearn_amd import ops

    if k_proj.shape != v_proj.shape:
        raise ValueError(f"{k_proj.shape=} != {v_proj.shape=}")
    if k_proj.shape[1] != key_positions.shape[1]:
        raise ValueError(f"{k_proj.shape[1]=} != {key_positions.shape[1]=}")
    if k_proj.shape[1] != 1:
        raise ValueError("Currently only support single time step.")
    ops.paged_kv_insert(k_pages, v_pages, k_proj[:, 0].to(k_pages.dtype), v_proj[:, 0].to(v_pages.dtype),
                        page_indices, key_positions.reshape(-1).contiguous())
    return k_pages, v_pages
