"""Return type of the dispatch (axlearn/common/flash_attention/attention_types.py:13-42)."""

from dataclasses import dataclass, field
from typing import Any, Callable


@dataclass
class FlashAttentionWithShardMapSpecs:
    """A kernel callable plus the extra per-argument sharding specs / tensors it wants threaded
    through the caller's shard_map.  The HIP kernels need none: both dicts stay empty."""

    fn: Callable
    additional_in_specs: dict[str, Any] = field(default_factory=dict)
    additional_kwargs: dict[str, Any] = field(default_factory=dict)
