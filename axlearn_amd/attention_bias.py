"""Typed attention biases: the mask algebra the kernels' callers speak.

Host-side mirror (torch tensors) of the parts of axlearn/common/attention_bias.py the attention
kernel path consumes: `NEG_INF` (:43), lazy composite biases (:215-318), `split` (:321-346), tensor,
bool, segment-id and mask-fn biases (:349-597), the causal / sliding-window masks (:652-700,
:771-790) and `bool_to_bias` (:862-873).  Biases stay symbolic so that a kernel can recognise
"causal", "sliding window w" and "segment ids" and never materialise a [T, S] tensor; `value()`
materialises only when a caller explicitly asks.
"""

from __future__ import annotations

import dataclasses
from typing import Callable, Iterable, Optional, Sequence, Type, TypeVar

import torch

Tensor = torch.Tensor
NEG_INF = -1e15  # attention_bias.py:43
B = TypeVar("B", bound="BaseAttentionBias")
MaskFn = Callable[[Tensor, Tensor], Tensor]


# ------------------------------------------------------------------------------------ mask fns


def causal_mask(query_position: Tensor, key_position: Tensor) -> Tensor:
    """True where the query may attend the key: q >= k (attention_bias.py:652-658)."""
    return query_position >= key_position


class _SlidingWindowCausalMask:
    """q >= k and q - k <= w: the query sees itself plus w keys to its left
    (attention_bias.py:771-790)."""

    def __init__(self, sliding_window_size: int):
        if sliding_window_size < 0:
            raise ValueError(f"{sliding_window_size=} must be a natural number.")
        self.sliding_window_size = int(sliding_window_size)

    def __call__(self, query_position: Tensor, key_position: Tensor) -> Tensor:
        return causal_mask(query_position, key_position) & (
            query_position - key_position <= self.sliding_window_size
        )


def sliding_window_causal_mask(sliding_window_size: int) -> MaskFn:
    return _SlidingWindowCausalMask(sliding_window_size)


def and_masks(*mask_fns: MaskFn) -> MaskFn:
    """Intersection of mask fns (attention_bias.py:758-768)."""

    def mask(query_position, key_position):
        result = mask_fns[0](query_position, key_position)
        for fn in mask_fns[1:]:
            result = result & fn(query_position, key_position)
        return result

    return mask


def or_masks(*mask_fns: MaskFn) -> MaskFn:
    """Union of mask fns (attention_bias.py:745-755)."""

    def mask(query_position, key_position):
        result = mask_fns[0](query_position, key_position)
        for fn in mask_fns[1:]:
            result = result | fn(query_position, key_position)
        return result

    return mask


def bool_to_bias(mask: Optional[Tensor]) -> Optional[Tensor]:
    """True -> 0, False -> NEG_INF (attention_bias.py:862-873)."""
    if mask is None:
        return None
    if mask.dtype != torch.bool:
        raise ValueError("mask must be a Boolean tensor.")
    return (~mask).to(torch.float32) * NEG_INF


def _make_bool_segment_mask(*, source_segments: Tensor, target_segments: Tensor) -> Tensor:
    """[batch, ..., T] vs [batch, ..., S] -> [batch, 1, ..., T, S] equality
    (attention_bias.py:876-882). Id 0 (padding) is compared like any other id."""
    eq = target_segments.unsqueeze(-1) == source_segments.unsqueeze(-2)
    return eq.unsqueeze(1)


def make_segment_mask(*, source_segments: Tensor, target_segments: Tensor) -> Tensor:
    return bool_to_bias(
        _make_bool_segment_mask(source_segments=source_segments, target_segments=target_segments)
    )


def make_causal_biases(seq_len: int) -> Tensor:
    pos = torch.arange(seq_len)
    return bool_to_bias(causal_mask(pos[:, None], pos[None, :]))


def make_sliding_window_causal_biases(seq_len: int, sliding_window_size: int) -> Tensor:
    pos = torch.arange(seq_len)
    return bool_to_bias(sliding_window_causal_mask(sliding_window_size)(pos[:, None], pos[None, :]))


# ------------------------------------------------------------------------------------ biases


@dataclasses.dataclass(eq=False)
class BaseAttentionBias:
    """A lazily evaluated additive logit bias of shape [batch|1, heads|1, target, source]."""

    dtype: Optional[torch.dtype] = dataclasses.field(default=None, kw_only=True)

    def _value(self) -> Optional[Tensor]:
        raise NotImplementedError(type(self))

    def _shape(self) -> Optional[tuple]:
        """Shape of `value()` without materialising it, or None if there is no value."""
        v = self._value()
        return None if v is None else tuple(self._broadcast_value(v).shape)

    def has_value(self) -> bool:
        return self._shape() is not None

    def eval_shape(self) -> tuple:
        shape = self._shape()
        if shape is None:
            raise ValueError("AttentionBias has no value.")
        return shape

    def value(self) -> Optional[Tensor]:
        value = self._value()
        if value is not None and self.dtype is not None:
            value = value.to(self.dtype)
        return self._broadcast_value(value)

    def astype(self, dtype: torch.dtype) -> "BaseAttentionBias":
        return dataclasses.replace(self, dtype=dtype)

    def __add__(self, other: "BaseAttentionBias") -> "CompositeAttentionBias":
        return CompositeAttentionBias([self, other])

    @classmethod
    def _broadcast_value(cls, value: Optional[Tensor]) -> Optional[Tensor]:
        if value is None or value.dim() == 4:
            return value
        if value.dim() == 2:
            return value[None, None]
        if value.dim() == 3:
            return value[:, None]
        raise ValueError(f"Invalid attention_logit_biases shape: {tuple(value.shape)}.")

    def bias_and_residual(self, cls: Type[B]) -> "BiasAndResidual":
        """Splits `self` into (a bias of type `cls` or None, the rest)."""
        if isinstance(self, cls):
            return BiasAndResidual(bias=self, residual=CompositeAttentionBias([]))
        return BiasAndResidual(bias=None, residual=self)

    @classmethod
    def from_sequence(cls, biases: Sequence["BaseAttentionBias"]) -> Optional["BaseAttentionBias"]:
        if not biases:
            return None
        shape = biases[0].eval_shape()
        for bias in biases:
            if not isinstance(bias, cls):
                raise TypeError(f"Got bias type {type(bias)}, not instance of {cls}.")
            if bias.eval_shape() != shape:
                raise ValueError(f"Got shape mismatch {bias.eval_shape()} != {shape}.")
        if len(biases) == 1:
            return biases[0]
        raise NotImplementedError(cls)


@dataclasses.dataclass(eq=False)
class BiasAndResidual(BaseAttentionBias):
    bias: Optional[BaseAttentionBias] = None
    residual: Optional[BaseAttentionBias] = None

    def _value(self) -> Optional[Tensor]:
        parts = ([self.bias] if self.bias is not None else []) + [self.residual]
        return CompositeAttentionBias(parts).value()

    def __iter__(self):
        return iter((self.bias, self.residual))


@dataclasses.dataclass(eq=False)
class CompositeAttentionBias(BaseAttentionBias):
    """Sum of member biases; members without a value are skipped (attention_bias.py:215-318)."""

    biases: Sequence[BaseAttentionBias] = dataclasses.field(default_factory=list)

    def _nonzero(self) -> list:
        return [b for b in self.biases if b is not None and b.has_value()]

    def _value(self) -> Optional[Tensor]:
        members = self._nonzero()
        if not members:
            return None
        total = 0.0
        for b in members:
            total = total + b.value()
        return total

    def _shape(self) -> Optional[tuple]:
        shapes = [b._shape() for b in self._nonzero()]  # pylint: disable=protected-access
        if not shapes:
            return None
        return tuple(torch.broadcast_shapes(*shapes))

    def __add__(self, other: BaseAttentionBias) -> "CompositeAttentionBias":
        return CompositeAttentionBias([self, other])

    def bias_and_residual(self, cls: Type[B]) -> BiasAndResidual:
        direct = super().bias_and_residual(cls)
        if direct.bias is not None:
            return direct
        pending = list(self._nonzero())
        found, rest = [], []
        while pending:
            member = pending.pop()
            part = member.bias_and_residual(cls)
            if part.bias is not None:
                found.append(part.bias)
                target = pending
            else:
                target = rest
            if part.residual.has_value():
                target.append(part.residual)
        return BiasAndResidual(bias=cls.from_sequence(found), residual=CompositeAttentionBias(rest))

    def _flatten(self) -> "CompositeAttentionBias":
        todo, flat = [self], []
        while todo:
            b = todo.pop()
            if isinstance(b, CompositeAttentionBias):
                todo.extend(b._nonzero())  # pylint: disable=protected-access
            else:
                flat.append(b)
        return CompositeAttentionBias(flat)


def split(bias: BaseAttentionBias, *cls: Type[BaseAttentionBias]) -> Iterable[BaseAttentionBias]:
    """Yields len(cls)+1 biases: one per requested type (ZeroAttentionBias if absent), then the
    residual; their sum equals `bias` (attention_bias.py:321-346)."""
    for c in cls:
        result, bias = bias.bias_and_residual(c)
        if isinstance(bias, cls):
            raise NotImplementedError("Got a residual of type in `cls`.")
        yield ZeroAttentionBias() if result is None else result
    yield bias


@dataclasses.dataclass(eq=False)
class TensorAttentionBias(BaseAttentionBias):
    """An explicit float bias tensor [batch|1, heads|1, target, source] (attention_bias.py:349-383)."""

    _internal_value: Optional[Tensor] = None

    def __post_init__(self):
        if self._internal_value is not None and self._internal_value.dim() != 4:
            raise ValueError(f"Invalid shape {tuple(self._internal_value.shape)}.")

    def _value(self) -> Tensor:
        return self._internal_value

    def _shape(self):
        return tuple(self._internal_value.shape)

    @classmethod
    def from_tensor(cls, tensor: Tensor) -> "TensorAttentionBias":
        return cls(cls._broadcast_value(tensor))


@dataclasses.dataclass(eq=False)
class BoolAttentionBias(BaseAttentionBias):
    """A bias given as a keep-mask (attention_bias.py:399-430)."""

    def _value(self) -> Optional[Tensor]:
        return bool_to_bias(self.bool_value())

    def bool_value(self) -> Optional[Tensor]:
        v = self._bool_value()
        if v is not None:
            v = v.to(torch.bool)
        return self._broadcast_value(v)

    def _bool_value(self) -> Optional[Tensor]:
        raise NotImplementedError(type(self))


@dataclasses.dataclass(eq=False)
class ZeroAttentionBias(BoolAttentionBias):
    """Adds nothing (attention_bias.py:723-742)."""

    def _bool_value(self) -> None:
        return None

    def _shape(self):
        return None

    def __eq__(self, other):
        return type(other) is type(self)

    __hash__ = None


@dataclasses.dataclass(eq=False)
class SegmentIdAttentionBias(BoolAttentionBias):
    """Packing mask: a query attends a key iff their segment ids are equal
    (attention_bias.py:433-459). segment_ids: [batch, seq_len] int."""

    segment_ids: Optional[Tensor] = None

    def _bool_value(self) -> Tensor:
        return _make_bool_segment_mask(
            target_segments=self.segment_ids, source_segments=self.segment_ids
        )

    def _shape(self):
        b, t = self.segment_ids.shape
        return (b, 1, t, t)


@dataclasses.dataclass(eq=False)
class MaskFnAttentionBias(BoolAttentionBias):
    """A keep-mask given by a function of (query position, key position)
    (attention_bias.py:501-597). target_positions [1|batch, T], source_positions [1|batch, S]."""

    mask: Optional[MaskFn] = None
    target_positions: Optional[Tensor] = dataclasses.field(default=None, kw_only=True)
    source_positions: Optional[Tensor] = dataclasses.field(default=None, kw_only=True)

    def _bool_value(self) -> Optional[Tensor]:
        tp, sp = self.target_positions, self.source_positions
        if tp.dim() != 2 or sp.dim() != 2:
            raise ValueError(f"{tuple(tp.shape)=} or {tuple(sp.shape)=} is not rank 2.")
        return self.mask(tp[:, :, None], sp[:, None, :])

    def _shape(self):
        tp, sp = self.target_positions, self.source_positions
        return (max(tp.shape[0], sp.shape[0]), 1, tp.shape[1], sp.shape[1])

    @classmethod
    def from_sequence(
        cls, biases: Sequence["MaskFnAttentionBias"]
    ) -> Optional["MaskFnAttentionBias"]:
        try:
            return super().from_sequence(biases)
        except NotImplementedError:
            pass
        # Several structured masks over the same positions: causal AND sliding(w1) AND sliding(w2)
        # is sliding(min w); keeping the structure lets a kernel still recognise the mask.
        pos = dict(
            target_positions=biases[0].target_positions,
            source_positions=biases[0].source_positions,
        )
        if all(isinstance(b, (CausalAttentionBias, SlidingWindowAttentionBias)) for b in biases):
            windows = [b.sliding_window_size for b in biases if isinstance(b, SlidingWindowAttentionBias)]
            if not windows:
                return biases[0]
            w = min(windows)
            return SlidingWindowAttentionBias(
                sliding_window_causal_mask(w), sliding_window_size=w, **pos
            )
        fns = [b.mask for b in biases]
        return MaskFnAttentionBias(and_masks(*fns), **pos)


@dataclasses.dataclass(eq=False)
class CausalAttentionBias(MaskFnAttentionBias):
    """Causal mask (attention_bias.py:661-680)."""

    mask: Optional[MaskFn] = causal_mask


@dataclasses.dataclass(eq=False)
class SlidingWindowAttentionBias(MaskFnAttentionBias):
    """Sliding-window causal mask; total window = sliding_window_size + 1
    (attention_bias.py:683-699)."""

    sliding_window_size: int = dataclasses.field(default=0, kw_only=True)


@dataclasses.dataclass(eq=False)
class BoolTensorAttentionBias(BoolAttentionBias):
    """An explicit boolean keep-mask tensor (attention_bias.py:600-631)."""

    _internal_bool_value: Optional[Tensor] = None

    def __post_init__(self):
        v = self._internal_bool_value
        if v is not None and v.dim() != 4:
            raise ValueError(f"Invalid shape {tuple(v.shape)}.")
        if v is not None and v.dtype != torch.bool:
            raise ValueError(f"Invalid dtype {v.dtype}, expected bool.")

    def _bool_value(self) -> Tensor:
        return self._internal_bool_value

    def _shape(self):
        return tuple(self._internal_bool_value.shape)

    @classmethod
    def from_tensor(cls, tensor: Tensor) -> "BoolTensorAttentionBias":
        return cls(cls._broadcast_value(tensor))


def as_attention_bias(bias) -> BaseAttentionBias:
    """None / float tensor / bias -> bias (attention_bias.py:634-649)."""
    if bias is None:
        return ZeroAttentionBias()
    if isinstance(bias, torch.Tensor):
        if not bias.dtype.is_floating_point:
            raise ValueError(f"bias must have a floating dtype, got {bias.dtype}.")
        return TensorAttentionBias.from_tensor(bias)
    if isinstance(bias, BaseAttentionBias):
        return bias
    raise NotImplementedError(type(bias))
