"""Flash-attention prefill / training kernels: the HIP replacement for the Pallas path.

Mirrors the kernel entry point `flash_attention(...)` (axlearn/common/flash_attention/
gpu_attention.py:250-287, custom VJP :428-430, :789) and the dispatch class
`PallasGPUFlashAttention` (:929-992).  Differences that follow from the machine mapping, not from
the mathematics:
  * KV heads are never repeated in memory: the kernels read the shared kv head (the reference
    repeats, :975-976, and lets autodiff sum dK/dV back);
  * structured masks (none / causal / sliding window, optionally with segment ids) are evaluated
    in closed form from block indices; any other `mask_fn` is materialised once as a dense 0 / -1e15
    bias `[1,1,T,S]` (what `MaskFnAttentionBias.value()` is) and takes the dense-bias kernels,
    instead of being traced into a block map;
  * dropout masks are drawn with torch's generator, not JAX's PRNG: the kernels take the mask as an
    input (as the Pallas kernel does, gpu_attention.py:374-385), so results agree with the reference
    for a given mask, not for a given key.
"""

from __future__ import annotations

import logging
from typing import Optional, Tuple

import torch

from axlearn_amd import ops
from axlearn_amd.attention_bias import (
    BaseAttentionBias,
    CausalAttentionBias,
    MaskFn,
    MaskFnAttentionBias,
    SegmentIdAttentionBias,
    SlidingWindowAttentionBias,
    _SlidingWindowCausalMask,
    bool_to_bias,
    causal_mask,
    split,
)
from axlearn_amd.config import config_class
from axlearn_amd.flash_attention.common import BaseFlashAttention, Nested, Tensor, get_segment_ids
from axlearn_amd.kv_cache import BaseKVCache, KVCache

FLASH_ATTN_RESIDUAL_NAME = "flash_residuals"


def classify_mask_fn(mask_fn: Optional[MaskFn]) -> Optional[Tuple[int, int]]:
    """Maps a mask fn to (mask_kind, window) if the kernels can evaluate it in closed form."""
    if mask_fn is None:
        return ops.MASK_NONE, 0
    if mask_fn is causal_mask:
        return ops.MASK_CAUSAL, 0
    if isinstance(mask_fn, _SlidingWindowCausalMask):
        return ops.MASK_SLIDING_WINDOW, mask_fn.sliding_window_size
    return None


def classify_mask_bias(mask: BaseAttentionBias) -> Optional[Tuple[int, int]]:
    if not mask.has_value():
        return ops.MASK_NONE, 0
    if isinstance(mask, SlidingWindowAttentionBias):
        return ops.MASK_SLIDING_WINDOW, int(mask.sliding_window_size)
    if isinstance(mask, CausalAttentionBias):
        return ops.MASK_CAUSAL, 0
    if isinstance(mask, MaskFnAttentionBias):
        return classify_mask_fn(mask.mask)
    return None


def padded_head_dim(head_dim: int) -> Optional[int]:
    """Compiled width the kernels run a given head dim at (None if it does not fit).

    The Pallas kernel pads the head dim to the next power of two inside its blocks and masks the
    extra columns (gpu_attention.py:172-176, :328).  The 16-bit HIP kernels do the same on the tensors
    as they are for any multiple of 8 (`runs_at_native_head_dim`); what they do not take that way is
    zero-padded to the width by `_pad_last` instead: zero columns of q/k add nothing to the logits and
    zero columns of v give zero output columns, which are sliced off again."""
    for width in (64, 128):
        if head_dim <= width:
            return width
    return None


def runs_at_native_head_dim(query: Tensor, key: Tensor, value: Tensor, *, aux: bool) -> bool:
    """Whether the kernels take these tensors without padded copies: head dims 64 and 128 always;
    other multiples of 8 in bf16 / f16 without a bias or dropout mask, rows at least one compiled
    width apart (the kernels' tile loads assume that much; a single head of 72 columns is not)."""
    head_dim = query.shape[-1]
    if head_dim in (64, 128):
        return True
    width = padded_head_dim(head_dim)
    if width is None or head_dim % 8 != 0 or aux or query.dtype == torch.float32:
        return False
    return all(x.stride(1) >= width and x.shape[2] * head_dim >= width for x in (query, key, value))


def _pad_last(x: Tensor, width: int) -> Tensor:
    return x if x.shape[-1] == width else torch.nn.functional.pad(x, (0, width - x.shape[-1]))


def get_dropout_mask(shape, *, prng_key, rate: float, device) -> Tensor:
    """Bool mask of `shape`, True = dropped with probability `rate` (layers.py:140-142).

    prng_key: a torch.Generator on `device`, or an int / integer tensor used as its seed."""
    if isinstance(prng_key, torch.Generator):
        gen = prng_key
    else:
        if prng_key is None:
            raise ValueError("prng_key must be provided when dropout_rate > 0.")
        seed = int(torch.as_tensor(prng_key).reshape(-1)[-1].item()) if not isinstance(prng_key, int) else prng_key
        gen = torch.Generator(device=device)
        gen.manual_seed(seed & 0x7FFFFFFFFFFFFFFF)
    return torch.rand(shape, generator=gen, device=device, dtype=torch.float32) < rate


def mask_fn_as_bias(mask_fn: MaskFn, q_len: int, kv_len: int, device, q_pos_offset: int = 0) -> Tensor:
    """An arbitrary mask fn as the dense bias `[1,1,T,S]` it stands for (attention_bias.py:862-873)."""
    qp = torch.arange(q_len, device=device)[:, None] + q_pos_offset
    kp = torch.arange(kv_len, device=device)[None, :]
    keep = torch.as_tensor(mask_fn(qp, kp), device=device).expand(q_len, kv_len)
    return bool_to_bias(keep)[None, None].to(torch.float32)


def _attend(query, key, value, segment_ids, softmax_scale, mask_kind, window, logit_sink=None,
            bias=None, dropout_mask=None, dropout_rate=0.0, save_residuals=True, bwd_ds_workspace=None,
            bwd_workspace_limit_bytes=None):
    """Pads the head dim if needed and runs the differentiable kernel pair."""
    head_dim = query.shape[-1]
    width = padded_head_dim(head_dim)
    if width is None:
        raise NotImplementedError(f"{head_dim=} > 128 is not supported by the HIP kernels.")
    if runs_at_native_head_dim(query, key, value, aux=bias is not None or dropout_mask is not None):
        width = head_dim
    out = _FlashAttentionFn.apply(
        _pad_last(query, width), _pad_last(key, width), _pad_last(value, width), segment_ids,
        softmax_scale, mask_kind, window, logit_sink, bias, dropout_mask, dropout_rate, save_residuals,
        bwd_ds_workspace, bwd_workspace_limit_bytes,
    )
    return out if width == head_dim else out[..., :head_dim]


class _FlashAttentionFn(torch.autograd.Function):
    """Forward = axl_flash_fwd, backward = axl_flash_bwd.

    The residuals (out, lse) are what the reference tags `flash_residuals` for its remat policies
    (gpu_attention.py:423, remat.py:13-58).  With save_residuals=False they are not kept: the
    backward re-runs the forward kernel on the saved q, k, v first, trading one forward pass for
    [B,T,Hq,D] + [B,Hq,T] of memory, and produces bit-identical gradients.  bwd_ds_workspace=True
    asks the backward to keep dS in its workspace (AXL_BWD_DS_WORKSPACE: about T*S bytes per (batch,
    head) more, 5 GEMMs instead of 7; ignored where that path does not apply), False to recompute dS
    in the dQ kernel, None to take the dS workspace whenever it fits bwd_workspace_limit_bytes (None:
    a sixteenth of the device's memory)."""

    @staticmethod
    def forward(ctx, query, key, value, segment_ids, softmax_scale, mask_kind, window, logit_sink,
                bias, dropout_mask, dropout_rate, save_residuals, bwd_ds_workspace=None,
                bwd_workspace_limit_bytes=None):
        aux = dict(bias=bias, dropout_mask=dropout_mask, dropout_rate=dropout_rate)
        out, lse = ops.flash_fwd(
            query, key, value, softmax_scale=softmax_scale, mask_kind=mask_kind,
            sliding_window=window, segment_ids=segment_ids, logit_sink=logit_sink, **aux,
        )
        if save_residuals:
            ctx.save_for_backward(query, key, value, out, lse, logit_sink)
        else:
            ctx.save_for_backward(query, key, value, None, None, logit_sink)
        ctx.segment_ids = segment_ids
        ctx.aux = aux  # not differentiated: the bias gets no gradient (gpu_attention.py:786)
        ctx.args = (softmax_scale, mask_kind, window)
        ctx.bwd_ds_workspace = None if bwd_ds_workspace is None else bool(bwd_ds_workspace)
        ctx.bwd_workspace_limit_bytes = bwd_workspace_limit_bytes
        return out

    @staticmethod
    def backward(ctx, d_out):
        query, key, value, out, lse, logit_sink = ctx.saved_tensors
        softmax_scale, mask_kind, window = ctx.args
        if out is None:  # residuals were not saved: recompute them
            out, lse = ops.flash_fwd(
                query, key, value, softmax_scale=softmax_scale, mask_kind=mask_kind,
                sliding_window=window, segment_ids=ctx.segment_ids, logit_sink=logit_sink, **ctx.aux,
            )
        if d_out.stride(-1) != 1:
            d_out = d_out.contiguous()
        grads = ops.flash_bwd(
            query, key, value, out, lse, d_out, softmax_scale=softmax_scale, mask_kind=mask_kind,
            sliding_window=window, segment_ids=ctx.segment_ids, logit_sink=logit_sink,
            ds_workspace=ctx.bwd_ds_workspace, ds_workspace_limit=ctx.bwd_workspace_limit_bytes, **ctx.aux,
        )
        d_sink = grads[3].to(logit_sink.dtype) if logit_sink is not None else None
        return grads[0], grads[1], grads[2], None, None, None, None, d_sink, None, None, None, None, None, None


# pylint: disable-next=too-many-positional-arguments
def flash_attention(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    bias: Optional[Tensor] = None,
    segment_ids: Optional[Tensor] = None,
    prng_key: Optional[Tensor] = None,
    softmax_scale: float = 1.0,
    mask_fn: Optional[MaskFn] = None,
    dropout_rate: float = 0.0,
    block_q: int = 128,
    block_k: int = 128,
    num_warps: Optional[int] = None,
    num_stages: Optional[int] = None,
    grid=None,
    interpret: bool = False,
    debug: bool = False,
) -> Tensor:
    """Differentiable flash attention; same signature as gpu_attention.py:250-267.

    query [B,T,Hq,D]; key/value [B,S,Hkv,D] (Hkv may be smaller than Hq); segment_ids [B,T].
    bias [B|1,Hq|1,T,S]: dense additive logit bias (no gradient).  dropout_rate > 0 draws a mask from
    `prng_key` (see `get_dropout_mask`).  The Pallas/Triton tuning arguments (block_q .. debug) are
    accepted and ignored: tiling is fixed by the HIP kernels.
    """
    del block_q, block_k, num_warps, num_stages, grid, debug
    if interpret:
        raise NotImplementedError("The HIP kernels have no interpret mode; they only run on the GPU.")
    if not 0.0 <= dropout_rate < 1.0:
        raise ValueError(f"Dropout rate must be in [0, 1). Got {dropout_rate=}")
    kind = classify_mask_fn(mask_fn)
    if kind is None:  # arbitrary mask fn: as a dense bias
        dense = mask_fn_as_bias(mask_fn, query.shape[1], key.shape[1], query.device)
        bias = dense if bias is None else bias.to(torch.float32) + dense
        kind = (ops.MASK_NONE, 0)
    dropout_mask = None
    if dropout_rate > 0.0:
        shape = (query.shape[0], query.shape[2], query.shape[1], key.shape[1])
        dropout_mask = get_dropout_mask(shape, prng_key=prng_key, rate=dropout_rate, device=query.device)
    return _attend(query, key, value, segment_ids, float(softmax_scale), kind[0], kind[1],
                   bias=bias, dropout_mask=dropout_mask, dropout_rate=float(dropout_rate))


class HipFlashAttention(BaseFlashAttention):
    """MI355X flash attention (forward + backward) behind the dispatch API.

    Takes the slot of `CuDNNGPUFlashAttention` / `PallasGPUFlashAttention`
    (axlearn/common/flash_attention/utils.py:41-50).

    With `kv_cache_type=KVCache` and more than one query row it serves incremental prefill: a chunk
    of queries per sequence, each chunk sitting at its own offset into the (contiguous) cache, as
    given by a causal / sliding-window bias with per-batch `target_positions`
    (utils_test.py:361-478).  That mode is forward only."""

    @config_class
    class Config(BaseFlashAttention.Config):
        # False: do not keep (out, lse) for the backward, recompute them there instead; the
        # counterpart of leaving `flash_residuals` out of the remat policy's saved names.
        save_residuals: bool = True
        # The backward can keep dS in its workspace (AXL_BWD_DS_WORKSPACE) where that path applies:
        # about T*S bytes per (batch, head) of transient memory for a backward that runs 5 GEMMs
        # instead of 7.  None (default): do so whenever that workspace fits bwd_workspace_limit_bytes;
        # True / False force the choice.  Also settable through backend_overrides["bwd_ds_workspace"].
        bwd_ds_workspace: Optional[bool] = None
        # Largest backward workspace the automatic choice may take; None = a sixteenth of the device's
        # memory (18 GB on an MI355X: C2 and C3 of the benchmark take the dS workspace, the 69 GB of a
        # 32768-token sequence do not).  Also settable through backend_overrides.
        bwd_workspace_limit_bytes: Optional[int] = None

    _kv_cache_type = None

    def _incremental_supported(self, input_batch: Nested) -> bool:
        query, key = input_batch["query"], input_batch["key"]
        if key.shape[1] % 128 != 0:
            return self._log_unsupported(f"{key.shape[1]=} is not divisible by 128")
        if self.cfg.dropout_rate != 0.0:
            raise ValueError("Dropout rate cannot be set for decoding!")
        mask, segment_ids, explicit_bias = split(input_batch["bias"], MaskFnAttentionBias, SegmentIdAttentionBias)
        if segment_ids.has_value() or explicit_bias.has_value():
            return self._log_unsupported("incremental prefill takes a causal or sliding-window mask only.")
        kind = classify_mask_bias(mask)
        if kind is None or kind[0] == ops.MASK_NONE or getattr(mask, "target_positions", None) is None:
            return self._log_unsupported("incremental prefill needs a causal / sliding-window mask with target_positions.")
        if mask.target_positions.shape[1] != query.shape[1]:
            return self._log_unsupported("target_positions do not match the query length.")
        return True

    def is_supported(self, input_batch: Nested, kv_cache_type: Optional[type[BaseKVCache]]) -> bool:
        if not super().is_supported(input_batch=input_batch, kv_cache_type=kv_cache_type):
            return False
        if kv_cache_type is not None and kv_cache_type != KVCache:
            return self._log_unsupported(f"{kv_cache_type=}")
        query, key = input_batch["query"], input_batch["key"]
        if kv_cache_type == KVCache:
            if not self._incremental_supported(input_batch):
                return False
        elif not self._check_block_size(input_batch=input_batch, block_size=128):
            return False
        self._kv_cache_type = kv_cache_type
        head_dim = query.shape[-1]
        if padded_head_dim(head_dim) is None:  # same limit as gpu_attention.py:954
            return self._log_unsupported(f"{head_dim=} > 128")
        if query.dtype not in (torch.bfloat16, torch.float16, torch.float32):
            return self._log_unsupported(f"{query.dtype=} (supported: bfloat16, float16, float32)")
        if key.dtype != query.dtype or input_batch["value"].dtype != query.dtype:
            return self._log_unsupported("query, key and value dtypes differ")
        logit_sink = input_batch.get("logit_sink", None)
        if logit_sink is not None and not logit_sink.is_cuda:
            return self._log_unsupported("logit sink is not on the GPU.")
        if not 0.0 <= self.cfg.dropout_rate < 1.0:
            raise ValueError(f"Dropout rate must be in [0, 1). Got {self.cfg.dropout_rate=}")
        if self.cfg.dropout_rate > 0.0 and input_batch.get("prng_key", None) is None:
            return self._log_unsupported("dropout needs input_batch['prng_key'].")
        if not (self.cfg.softmax_scale > 0.0):
            return self._log_unsupported(f"{self.cfg.softmax_scale=} must be positive")
        bias: BaseAttentionBias = input_batch["bias"]
        _, segment_ids, _ = split(bias, MaskFnAttentionBias, SegmentIdAttentionBias)
        if segment_ids.has_value() and query.shape[1] != key.shape[1]:
            return self._log_unsupported("segment ids need identical query and key lengths.")
        if not query.is_cuda:
            return self._log_unsupported("tensors are not on the GPU.")
        return True

    def _incremental_prefill(self, input_batch: Nested) -> Tensor:
        """Queries at per-sequence offsets into the cache; rows padded up to the 128-row block."""
        query, key, value = input_batch["query"], input_batch["key"], input_batch["value"]
        mask, _, _ = split(input_batch["bias"], MaskFnAttentionBias, SegmentIdAttentionBias)
        kind = classify_mask_bias(mask)
        b, t, _, head_dim = query.shape
        positions = mask.target_positions.to(query.device)
        offsets = positions[:, 0].to(torch.int32).expand(b).contiguous()
        consecutive = positions[:, :1] + torch.arange(t, device=query.device)[None]
        if not torch.equal(positions, consecutive.to(positions.dtype)):
            raise NotImplementedError("target_positions of a chunk must be consecutive.")
        width = head_dim if runs_at_native_head_dim(query, key, value, aux=False) else padded_head_dim(head_dim)
        rows = -(-t // 128) * 128
        q = torch.nn.functional.pad(query.detach(), (0, width - head_dim, 0, 0, 0, rows - t))
        out, _ = ops.flash_fwd(
            q, _pad_last(key.detach(), width), _pad_last(value.detach(), width),
            softmax_scale=float(self.cfg.softmax_scale), mask_kind=kind[0], sliding_window=kind[1],
            q_pos_offsets=offsets, logit_sink=input_batch.get("logit_sink", None), return_lse=False,
        )
        return out[:, :t, :, :head_dim]

    def __call__(self, input_batch: Nested) -> Tensor:
        if self._kv_cache_type == KVCache:
            return self._incremental_prefill(input_batch)
        query, key, value = input_batch["query"], input_batch["key"], input_batch["value"]
        bias: BaseAttentionBias = input_batch["bias"]
        mask, segment_ids, explicit_bias = split(bias, MaskFnAttentionBias, SegmentIdAttentionBias)
        dense = explicit_bias.value() if explicit_bias.has_value() else None  # [B|1,H|1,T,S]
        kind = classify_mask_bias(mask)
        if kind is None:  # a mask fn the kernels have no closed form for: its dense value
            mask_bias = mask.value().to(torch.float32)
            dense = mask_bias if dense is None else dense.to(torch.float32) + mask_bias
            kind = (ops.MASK_NONE, 0)
        if dense is not None:
            dense = dense.to(query.device)
        seg = get_segment_ids(query=query, key=key, segment_ids=segment_ids)
        rate = float(self.cfg.dropout_rate)
        dropout_mask = None
        if rate > 0.0:
            shape = (query.shape[0], query.shape[2], query.shape[1], key.shape[1])
            dropout_mask = get_dropout_mask(shape, prng_key=input_batch.get("prng_key", None), rate=rate,
                                            device=query.device)
        logging.info("HipFlashAttention: mask_kind=%d window=%d segment_ids=%s dense_bias=%s dropout=%g",
                     kind[0], kind[1], seg is not None, dense is not None, rate)
        return _attend(
            query, key, value, seg, float(self.cfg.softmax_scale), kind[0], kind[1],
            input_batch.get("logit_sink", None), bias=dense, dropout_mask=dropout_mask, dropout_rate=rate,
            save_residuals=bool(self.get_backend_overrides("save_residuals", self.cfg.save_residuals)),
            bwd_ds_workspace=self.get_backend_overrides("bwd_ds_workspace", self.cfg.bwd_ds_workspace),
            bwd_workspace_limit_bytes=self.get_backend_overrides(
                "bwd_workspace_limit_bytes", self.cfg.bwd_workspace_limit_bytes),
        )
