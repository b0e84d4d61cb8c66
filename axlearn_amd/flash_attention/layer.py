"""The layer-level caller of the attention kernels, and its two config modifiers.

`FlashAttention.compute_attention` repeats what `FlashAttention._compute_attention` does on one
device (axlearn/common/flash_attention/layer.py:218-376), in the same order:

  1. the logit bias is cast to the dtype of the query projections (:253);
  2. `softmax_scale` defaults to 1.0, because the layer has already folded the scale into q
     (`scale_query`) before it gets here (:260);
  3. `flash_attention_implementation` picks a kernel; `None` means none supports the request and the
     caller's standard attention runs instead (:278-285);
  4. the kernel is called on the `input_batch` dictionary {query, key, value, prng_key, bias,
     logit_sink, page_tables} plus whatever extra arguments the kernel's `build` asked for (:356-365);
  5. the result is `(context, probs)` where `probs` has the shape [batch, heads, target, source] and no
     contents (`jnp.empty`, :371-375): here a tensor on torch's "meta" device, which has a shape and no
     storage.

The sharding steps of the original (`maybe_shard`, `shard_map`, the per-device PRNG keys, :296-354)
have no counterpart on one GPU and are left out; `_maybe_repeat_kv_heads` (:182-216) only repeats kv
heads to make them divisible by a mesh axis, so it is the identity here.

`FlashBlockSizeModifier` and `BackendOverrideModifier` (layer.py:434-496) rewrite every
`FlashAttention.Config` found in a config tree.
"""

from __future__ import annotations

import dataclasses
from typing import Any, Callable, Optional

import torch

from axlearn_amd.attention_bias import BaseAttentionBias
from axlearn_amd.config import Configurable, config_class
from axlearn_amd.flash_attention.utils import flash_attention_implementation
from axlearn_amd.kv_cache import BaseKVCache

Tensor = torch.Tensor


class FlashAttention(Configurable):
    """The part of the reference's `FlashAttention` layer that sits directly above the kernels."""

    @config_class
    class Config(Configurable.Config):
        # Scale of the logits; None = 1.0, the query projections are expected to be scaled (layer.py:260).
        softmax_scale: Optional[float] = None
        # Block sizes handed to the dispatch (layer.py:68-75); gpu_block_size None = 128 (:272).
        tpu_block_size: int = 512
        gpu_block_size: Optional[int] = None
        # Kernel-specific settings, e.g. {"save_residuals": False} (layer.py:81).
        backend_overrides: Optional[dict] = None
        dropout_rate: float = 0.0
        backend: str = "gpu"

    def compute_attention(
        self,
        *,
        q_proj: Tensor,
        k_proj: Tensor,
        v_proj: Tensor,
        attention_logit_biases: BaseAttentionBias,
        page_indices: Optional[Tensor] = None,
        kv_cache_type: Optional[type[BaseKVCache]] = None,
        logit_sink: Optional[Tensor] = None,
        prng_key: Optional[torch.Generator] = None,
        is_training: bool = False,
        fallback: Optional[Callable[..., tuple[Tensor, Tensor]]] = None,
    ) -> tuple[Tensor, Tensor]:
        """q_proj [B,T,Hq,D]; k_proj / v_proj [B,S,Hkv,D], or page pools [Hkv,pages,page,D] with
        page_indices [B,pages_per_seq].  Returns (context [B,T,Hq,D], probs [B,Hq,T,S] without contents).

        `fallback(q_proj=, k_proj=, v_proj=, attention_logit_biases=, page_indices=, logit_sink=)` stands
        for the base layer's standard attention, which the reference calls when no kernel supports the
        request (layer.py:278-285).  This package computes nothing outside its HIP kernels: without a
        fallback such a request raises."""
        cfg = self.config
        attention_logit_biases = attention_logit_biases.astype(q_proj.dtype)
        softmax_scale = cfg.softmax_scale if cfg.softmax_scale is not None else 1.0
        flash_specs = flash_attention_implementation(
            backend=cfg.backend,
            query=q_proj,
            key=k_proj,
            value=v_proj,
            bias=attention_logit_biases,
            logit_sink=logit_sink,
            softmax_scale=softmax_scale,
            kv_cache_type=kv_cache_type,
            tpu_block_size=cfg.tpu_block_size,
            gpu_block_size=cfg.gpu_block_size or 128,
            dropout_rate=cfg.dropout_rate if is_training else 0.0,
            page_tables=page_indices,
            backend_overrides=cfg.backend_overrides,
        )
        if flash_specs is None:
            if fallback is None:
                raise NotImplementedError(
                    "no HIP attention kernel supports this request (see the 'Not using ...' log lines) and no "
                    "fallback attention was given; axlearn_amd has no non-HIP execution path of its own")
            return fallback(q_proj=q_proj, k_proj=k_proj, v_proj=v_proj, attention_logit_biases=attention_logit_biases,
                            page_indices=page_indices, logit_sink=logit_sink)
        batch, target_len, num_heads, _ = q_proj.shape
        source_len = k_proj.shape[1] if page_indices is None else k_proj.shape[2] * page_indices.shape[-1]
        input_batch = {
            "query": q_proj,
            "key": k_proj,
            "value": v_proj,
            "prng_key": prng_key,
            "bias": attention_logit_biases,
            "logit_sink": logit_sink,
            "page_tables": page_indices,
            **flash_specs.additional_kwargs,
        }
        outputs = flash_specs.fn(input_batch)
        output_probs = torch.empty((batch, num_heads, target_len, source_len), device="meta")
        return outputs, output_probs


def _visit_flash_configs(node: Any, fn: Callable[["FlashAttention.Config"], None], seen: set) -> None:
    """Calls fn on every `FlashAttention.Config` reachable from `node` through dataclass fields, dicts,
    lists and tuples; does not descend into a `FlashAttention.Config` (layer.py:458-459 `enter_fn`)."""
    if id(node) in seen:
        return
    seen.add(id(node))
    if isinstance(node, FlashAttention.Config):
        fn(node)
        return
    if dataclasses.is_dataclass(node) and not isinstance(node, type):
        for f in dataclasses.fields(node):
            _visit_flash_configs(getattr(node, f.name), fn, seen)
    elif isinstance(node, dict):
        for v in node.values():
            _visit_flash_configs(v, fn, seen)
    elif isinstance(node, (list, tuple)):
        for v in node:
            _visit_flash_configs(v, fn, seen)


class FlashBlockSizeModifier(Configurable):
    """Sets tpu_block_size / gpu_block_size of every FlashAttention config in a tree (layer.py:434-462)."""

    @config_class
    class Config(Configurable.Config):
        tpu_block_size: Optional[int] = 512
        gpu_block_size: Optional[int] = None

    def __call__(self, cfg: Any) -> Any:
        tpu_block_size, gpu_block_size = self.config.tpu_block_size, self.config.gpu_block_size

        def visit(value: FlashAttention.Config):
            value.tpu_block_size = tpu_block_size
            value.gpu_block_size = gpu_block_size

        _visit_flash_configs(cfg, visit, set())
        return cfg


class BackendOverrideModifier(Configurable):
    """Merges `backend_overrides` into every FlashAttention config in a tree (layer.py:465-496):
    existing keys are updated, keys whose value is falsy (None) are not inserted."""

    @config_class
    class Config(Configurable.Config):
        backend_overrides: Optional[dict] = None

    def __call__(self, cfg: Any) -> Any:
        backend_overrides = self.config.backend_overrides

        def visit(value: FlashAttention.Config):
            if backend_overrides:
                if value.backend_overrides is None:
                    value.backend_overrides = dict()
                for override_key, override_value in backend_overrides.items():
                    if override_value:
                        value.backend_overrides.update({override_key: override_value})

        _visit_flash_configs(cfg, visit, set())
        return cfg
