"""CPU-only tests: mask algebra, block maps, kernel-class support gates, dispatch, and that the C-ABI
library loads and exports every symbol include/axl_attn.h declares.  No kernel is launched here."""

import ctypes
import json
import os
import re

import numpy as np
import pytest
import torch

from axlearn_amd import _lib
from axlearn_amd import attention_bias as ab
from axlearn_amd.flash_attention import common
from axlearn_amd.flash_attention.hip_attention import (
    HipFlashAttention,
    classify_mask_bias,
    classify_mask_fn,
    flash_attention,
)
from axlearn_amd.flash_attention.hip_decoding import HipDecoding, HipPagedAttention
from axlearn_amd.flash_attention.utils import (
    BACKENDS,
    PAGED_ATTN_BACKENDS,
    flash_attention_implementation,
)
from axlearn_amd.kv_cache import KVCache, PagedKVCache
from axlearn_amd import ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ----------------------------------------------------------------------------- mask algebra


def test_mask_tables_from_reference_tests(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "mask_tables.json")))
    for case in g["sliding_window_5x5"]:
        fn = ab.sliding_window_causal_mask(case["left_context"])
        got = fn(torch.arange(5)[:, None], torch.arange(5)[None, :]).int().tolist()
        assert got == case["expected"]
    for case in g["sliding_window2_with_time_step_3x5"]:
        fn = ab.sliding_window_causal_mask(2)
        got = fn(torch.arange(3)[:, None] + case["time_step"], torch.arange(5)[None, :]).int().tolist()
        assert got == case["expected"]
    assert ab.causal_mask(torch.arange(3)[:, None], torch.arange(3)[None, :]).int().tolist() == g["causal_3x3"]
    seg = g["segment_4x4"]
    bias = ab.make_segment_mask(target_segments=torch.tensor(seg["target_segments"]),
                                source_segments=torch.tensor(seg["source_segments"]))
    assert (bias == 0).int().tolist() == seg["expected"]
    assert float(bias.min()) == pytest.approx(-1e15)
    with pytest.raises(ValueError):
        ab.sliding_window_causal_mask(-1)


def test_composite_bias_and_split():
    t = 6
    pos = dict(target_positions=torch.arange(t)[None], source_positions=torch.arange(t)[None])
    seg_ids = torch.tensor([[1, 1, 1, 2, 2, 0]])
    dense = torch.randn(1, 1, t, t)
    bias = ab.CompositeAttentionBias(
        [ab.CausalAttentionBias(**pos), ab.SegmentIdAttentionBias(seg_ids), ab.TensorAttentionBias(dense)]
    )
    assert bias.eval_shape() == (1, 1, t, t)
    mask, seg, rest = ab.split(bias, ab.MaskFnAttentionBias, ab.SegmentIdAttentionBias)
    assert isinstance(mask, ab.CausalAttentionBias) and isinstance(seg, ab.SegmentIdAttentionBias)
    assert rest.has_value()
    total = mask.value() + seg.value() + rest.value()
    torch.testing.assert_close(total, bias.value())
    # Doubly masked element carries -2e15: biases are summed, not min-ed.
    assert float(bias.value()[0, 0, 0, 5]) < -1.5e15
    # Absent types come back as ZeroAttentionBias.
    m2, s2, r2 = ab.split(ab.CompositeAttentionBias([ab.TensorAttentionBias(dense)]),
                          ab.MaskFnAttentionBias, ab.SegmentIdAttentionBias)
    assert not m2.has_value() and not s2.has_value() and r2.has_value()
    assert isinstance(m2, ab.ZeroAttentionBias) and m2 == ab.ZeroAttentionBias()
    assert not ab.CompositeAttentionBias([]).has_value()
    with pytest.raises(ValueError):
        ab.CompositeAttentionBias([]).eval_shape()


def test_structured_masks_combine():
    t = 8
    pos = dict(target_positions=torch.arange(t)[None], source_positions=torch.arange(t)[None])
    mk = lambda w: ab.SlidingWindowAttentionBias(ab.sliding_window_causal_mask(w), sliding_window_size=w, **pos)
    bias = ab.CompositeAttentionBias([ab.CausalAttentionBias(**pos), mk(5), mk(3)])
    mask, rest = ab.split(bias, ab.MaskFnAttentionBias)
    assert not rest.has_value()
    assert classify_mask_bias(mask) == (ops.MASK_SLIDING_WINDOW, 3)
    torch.testing.assert_close(mask.value(), mk(3).value())
    assert classify_mask_fn(None) == (ops.MASK_NONE, 0)
    assert classify_mask_fn(ab.causal_mask) == (ops.MASK_CAUSAL, 0)
    assert classify_mask_fn(ab.sliding_window_causal_mask(7)) == (ops.MASK_SLIDING_WINDOW, 7)
    assert classify_mask_fn(lambda q, k: q == k) is None
    # A generic mask fn next to a causal one collapses to an opaque AND.
    generic = ab.MaskFnAttentionBias(lambda q, k: (q - k) % 2 == 0, **pos)
    mask, _ = ab.split(ab.CompositeAttentionBias([ab.CausalAttentionBias(**pos), generic]), ab.MaskFnAttentionBias)
    assert classify_mask_bias(mask) is None
    want = ab.causal_mask(torch.arange(t)[:, None], torch.arange(t)[None]) & ((torch.arange(t)[:, None] - torch.arange(t)[None]) % 2 == 0)
    assert torch.equal(mask.bool_value()[0, 0], want)


def test_as_attention_bias():
    assert isinstance(ab.as_attention_bias(None), ab.ZeroAttentionBias)
    assert isinstance(ab.as_attention_bias(torch.zeros(2, 2)), ab.TensorAttentionBias)
    with pytest.raises(ValueError):
        ab.as_attention_bias(torch.zeros(2, 2, dtype=torch.int32))
    with pytest.raises(ValueError):
        ab.bool_to_bias(torch.zeros(2, 2))


# ----------------------------------------------------------------------------- block maps


def test_block_maps(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "mask_tables.json")))["sliding_window_block_map_invariant"]
    for w in g["sliding_window_sz"]:
        for t in g["seq_len"]:
            for blk in g["block_size"]:
                kw = dict(q_seq_len=t, kv_seq_len=t, block_q=blk, block_k=blk)
                a = common.build_mask(ab.sliding_window_causal_mask(w), **kw)
                b = common.build_sliding_window_mask(**kw, sliding_window_size=w)
                assert (a == b).all(), (w, t, blk)
    # Brute force "tile keeps any element", unequal blocks.
    fn = ab.sliding_window_causal_mask(37)
    t, bq, bk = 256, 32, 64
    got = common.build_mask(fn, q_seq_len=t, kv_seq_len=t, block_q=bq, block_k=bk)
    full = fn(torch.arange(t)[:, None], torch.arange(t)[None, :]).numpy()
    want = full.reshape(t // bq, bq, t // bk, bk).any(axis=(1, 3))
    assert (got == want).all()
    assert (common.build_sliding_window_mask(q_seq_len=t, kv_seq_len=t, block_q=bq, block_k=bk, sliding_window_size=37) == want).all()
    info = common.query_iterator_indices(want)
    for i in range(want.shape[0]):
        n = info.kv_block_offset_size[i]
        assert list(info.kv_block_offset[i, :n]) == list(np.nonzero(want[i])[0])
    off, size = common.key_value_iterator_indices(want)
    for j in range(want.shape[1]):
        assert list(off[j, : size[j]]) == list(np.nonzero(want[:, j])[0])


def test_kernel_tile_ranges_match_block_map():
    """The closed-form key range the forward kernel iterates (128-row query block, 64-key tiles)
    covers exactly the live tiles of the reference's block map."""
    t, window = 1024, 300
    live = common.build_mask(ab.sliding_window_causal_mask(window), q_seq_len=t, kv_seq_len=t, block_q=128, block_k=64)
    for qb in range(t // 128):
        k_end = min(t, qb * 128 + 128)
        k_begin = max(0, qb * 128 - window)
        rng = set(range(k_begin // 64, (k_end + 63) // 64))
        assert rng == set(np.nonzero(live[qb])[0])


# ----------------------------------------------------------------------------- support gates


def _batch(t=128, s=128, hq=4, hkv=2, d=128, dtype=torch.bfloat16, bias=None, b=2):
    pos = dict(target_positions=torch.arange(t)[None], source_positions=torch.arange(s)[None])
    return dict(
        query=torch.zeros(b, t, hq, d, dtype=dtype), key=torch.zeros(b, s, hkv, d, dtype=dtype),
        value=torch.zeros(b, s, hkv, d, dtype=dtype),
        bias=bias if bias is not None else ab.CompositeAttentionBias([ab.CausalAttentionBias(**pos)]),
    )


def test_is_supported_raises_on_illogical_shapes():
    fa = HipFlashAttention.default_config().instantiate()
    bad = _batch()
    bad["key"] = torch.zeros(3, 128, 2, 128, dtype=torch.bfloat16)
    bad["value"] = bad["key"]
    with pytest.raises(ValueError, match="batch size"):
        fa.is_supported(bad, kv_cache_type=None)
    bad = _batch(hq=5, hkv=2)
    with pytest.raises(ValueError, match="divisible"):
        fa.is_supported(bad, kv_cache_type=None)
    bad = _batch()
    bad["value"] = torch.zeros(2, 64, 2, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        fa.is_supported(bad, kv_cache_type=None)
    bad = _batch()
    del bad["bias"]
    with pytest.raises(ValueError):
        fa.is_supported(bad, kv_cache_type=None)
    dec = HipDecoding.default_config().set(dropout_rate=0.1).instantiate()
    with pytest.raises(ValueError, match="Dropout"):
        dec.is_supported(_batch(t=1), kv_cache_type=KVCache)


def test_is_supported_returns_false_when_merely_unsupported(caplog):
    fa = HipFlashAttention.default_config().instantiate()
    assert not fa.is_supported(_batch(t=100, s=100), kv_cache_type=None)  # not a multiple of 128
    assert not fa.is_supported(_batch(dtype=torch.float16), kv_cache_type=None)
    assert not fa.is_supported(_batch(), kv_cache_type=PagedKVCache)
    assert not fa.is_supported(_batch(s=100), kv_cache_type=KVCache)  # cache length not a multiple of 128
    assert not fa.is_supported(_batch(d=136), kv_cache_type=None)  # head_dim > 128, gpu_attention.py:954
    # Dropout needs a key to draw the mask from; an impossible rate is an error, not "unsupported".
    assert not HipFlashAttention.default_config().set(dropout_rate=0.1).instantiate().is_supported(_batch(), None)
    with pytest.raises(ValueError, match="Dropout rate"):
        HipFlashAttention.default_config().set(dropout_rate=1.5).instantiate().is_supported(_batch(), None)
    # Everything fine except the tensors live on the CPU.
    assert not fa.is_supported(_batch(), kv_cache_type=None)
    assert fa.name() == "HipFlashAttention"
    assert fa.get_backend_overrides("x", 3) == 3
    dec = HipDecoding.default_config().instantiate()
    assert not dec.is_supported(_batch(t=2), kv_cache_type=KVCache)
    assert not dec.is_supported(_batch(t=1), kv_cache_type=None)
    paged = HipPagedAttention.default_config().instantiate()
    pb = _batch(t=1)
    with pytest.raises(ValueError):
        paged.is_supported(pb, kv_cache_type=PagedKVCache)  # no page_tables
    pb["page_tables"] = torch.zeros(2, 4, dtype=torch.int32)
    assert not paged.is_supported(pb, kv_cache_type=KVCache)


def test_dispatch_tables_and_fallback():
    assert BACKENDS["gpu"] == [HipDecoding, HipFlashAttention]
    assert PAGED_ATTN_BACKENDS["gpu"] == [HipPagedAttention]
    b = _batch()
    # CPU tensors / unknown backends: no kernel matches -> None (caller falls back to plain attention).
    assert flash_attention_implementation("gpu", query=b["query"], key=b["key"], value=b["value"], bias=b["bias"]) is None
    assert flash_attention_implementation("cpu", query=b["query"], key=b["key"], value=b["value"], bias=b["bias"]) is None
    assert flash_attention_implementation("tpu", query=b["query"], key=b["key"], value=b["value"], bias=b["bias"], dropout_rate=None) is None


def test_entry_point_rejects_what_kernels_cannot_do():
    q = torch.zeros(1, 128, 1, 128, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError):
        flash_attention(q, q, q, interpret=True)
    with pytest.raises(ValueError, match="Dropout rate"):
        flash_attention(q, q, q, dropout_rate=1.0)
    with pytest.raises(ValueError, match="prng_key"):
        flash_attention(q, q, q, dropout_rate=0.5)  # a mask cannot be drawn without a key
    with pytest.raises(NotImplementedError, match="128"):
        big = torch.zeros(1, 128, 1, 256, dtype=torch.bfloat16)
        flash_attention(big, big, big)
    # CPU tensors: there is no CPU path, whatever the optional inputs are.
    with pytest.raises(_lib.AxlError):
        flash_attention(q, q, q)
    with pytest.raises(_lib.AxlError):
        flash_attention(q, q, q, bias=torch.zeros(1, 1, 128, 128))
    with pytest.raises(_lib.AxlError):
        flash_attention(q, q, q, mask_fn=lambda a, b: a == b)


def test_arbitrary_mask_fn_and_dropout_mask_helpers():
    from axlearn_amd.flash_attention.hip_attention import get_dropout_mask, mask_fn_as_bias, padded_head_dim

    bias = mask_fn_as_bias(lambda a, b: (a - b) % 3 == 0, 4, 5, "cpu", q_pos_offset=1)
    assert bias.shape == (1, 1, 4, 5) and bias.dtype == torch.float32
    want = torch.tensor([[(t + 1 - s) % 3 == 0 for s in range(5)] for t in range(4)])
    assert torch.equal(bias[0, 0] == 0, want) and torch.equal(bias[0, 0] == ab.NEG_INF, ~want)
    m1 = get_dropout_mask((2, 3, 8, 16), prng_key=7, rate=0.4, device="cpu")
    m2 = get_dropout_mask((2, 3, 8, 16), prng_key=torch.tensor([0, 7]), rate=0.4, device="cpu")
    m3 = get_dropout_mask((2, 3, 8, 16), prng_key=8, rate=0.4, device="cpu")
    assert m1.dtype == torch.bool and torch.equal(m1, m2) and not torch.equal(m1, m3)
    assert 0.25 < m1.float().mean() < 0.55
    assert [padded_head_dim(d) for d in (8, 64, 65, 128, 129)] == [64, 64, 128, 128, None]


def test_config_protocol():
    cfg = HipFlashAttention.default_config().set(softmax_scale=0.5, gpu_block_size=64)
    inst = cfg.instantiate()
    assert inst.cfg.softmax_scale == 0.5 and inst.cfg.gpu_block_size == 64
    with pytest.raises(AttributeError):
        cfg.set(no_such_field=1)
    assert HipPagedAttention.default_config().sparse_ratio == 0.8


# ----------------------------------------------------------------------------- C ABI (no launches)


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "axl_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(axl_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    declared = _declared_functions()
    assert set(declared) == set(_lib.EXPORTED_SYMBOLS)
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name
    header = open(os.path.join(ROOT, "include", "axl_attn.h")).read()
    declared_version = int(re.search(r"#define AXL_ATTN_ABI_VERSION (\d+)", header).group(1))
    assert lib.axl_abi_version() == declared_version == _lib.ABI_VERSION
    assert lib.axl_last_error() is not None


def test_struct_layouts_match_header():
    """Field order of the ctypes mirrors equals the order in the header."""
    text = open(os.path.join(ROOT, "include", "axl_attn.h")).read()
    for cls in (_lib.AxlAttnAux, _lib.AxlFlashFwdParams, _lib.AxlFlashBwdParams, _lib.AxlDecodeBias,
                _lib.AxlPagedDecodeParams, _lib.AxlDecodeParams, _lib.AxlPageInsertParams):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cls.__name__, cls.__name__), text, flags=re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        names = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            for part in decl.split(","):
                names.append(re.findall(r"[A-Za-z_][A-Za-z_0-9]*", part)[-1])
        assert names == [f[0] for f in cls._fields_], cls.__name__


def test_abi_validation_without_gpu():
    """Argument checks run before any launch, so they are testable on a machine without a GPU."""
    lib = _lib.load()
    assert lib.axl_flash_fwd(None, None) == _lib.AXL_ERR_INVALID_ARGUMENT
    s = _lib.AxlStrides(1 << 20, 1024, 128)
    p = _lib.AxlFlashFwdParams(q=256, k=256, v=256, out=256, lse=None, segment_ids=None, q_strides=s, k_strides=s,
                               v_strides=s, out_strides=s, batch=1, q_len=128, kv_len=128, num_q_heads=3,
                               num_kv_heads=2, head_dim=128, dtype=0, mask_kind=1, sliding_window=0,
                               q_pos_offset=0, softmax_scale=1.0)
    assert lib.axl_flash_fwd(ctypes.byref(p), None) == _lib.AXL_ERR_INVALID_ARGUMENT
    assert b"divisible" in lib.axl_last_error()
    p.num_q_heads = 4
    p.head_dim = 76   # bf16: multiples of 8 up to 128 run on the tensors as they are, others do not
    assert lib.axl_flash_fwd(ctypes.byref(p), None) == _lib.AXL_ERR_UNSUPPORTED
    p.head_dim = 72   # ... if the rows lie at least one compiled width (128) apart
    p.k_strides = _lib.AxlStrides(1 << 20, 72, 72)
    assert lib.axl_flash_fwd(ctypes.byref(p), None) == _lib.AXL_ERR_UNSUPPORTED
    assert b"128 elements apart" in lib.axl_last_error()
    p.k_strides = s
    p.aux = _lib.AxlAttnAux(bias=256, bias_batch_stride=0, bias_head_stride=0, bias_row_stride=128, bias_dtype=1)
    assert lib.axl_flash_fwd(ctypes.byref(p), None) == _lib.AXL_ERR_UNSUPPORTED  # no such form with a bias
    p.aux = _lib.AxlAttnAux()
    p.dtype = 1       # float32: the compiled widths only
    assert lib.axl_flash_fwd(ctypes.byref(p), None) == _lib.AXL_ERR_UNSUPPORTED
    p.dtype = 0
    p.head_dim = 128
    p.q_len = 100
    assert lib.axl_flash_fwd(ctypes.byref(p), None) == _lib.AXL_ERR_UNSUPPORTED
    p.q_len = 128
    p.softmax_scale = 0.0
    assert lib.axl_flash_fwd(ctypes.byref(p), None) == _lib.AXL_ERR_INVALID_ARGUMENT
    p.softmax_scale = 1.0
    p.q = None
    assert lib.axl_flash_fwd(ctypes.byref(p), None) == _lib.AXL_ERR_INVALID_ARGUMENT
    p.q = 257
    assert lib.axl_flash_fwd(ctypes.byref(p), None) == _lib.AXL_ERR_UNSUPPORTED  # misaligned
    p.q = 256
    p.segment_ids = 256
    p.kv_len = 256
    assert lib.axl_flash_fwd(ctypes.byref(p), None) == _lib.AXL_ERR_INVALID_ARGUMENT  # seg needs T == S
    # Backward: workspace too small.
    bp = _lib.AxlFlashBwdParams(q=256, k=256, v=256, out=256, d_out=256, lse=256, dq=256, dk=256, dv=256,
                                segment_ids=None, q_strides=s, k_strides=s, v_strides=s, out_strides=s,
                                d_out_strides=s, dq_strides=s, dk_strides=s, dv_strides=s, batch=2, q_len=256,
                                kv_len=256, num_q_heads=4, num_kv_heads=2, head_dim=128, dtype=0, mask_kind=1,
                                sliding_window=0, q_pos_offset=0, softmax_scale=1.0, workspace=256, workspace_bytes=16)
    # delta and scaled lse, fp32 [B, Hq, T] each, plus the slack for rounding a 16-byte aligned pointer up to 256
    stats = 2 * (2 * 4 * 256 * 4) + 240
    assert lib.axl_flash_bwd_workspace_bytes(ctypes.byref(bp)) == stats
    # plain causal attention with the dS workspace: A = T / 128 = 2 -> 8 A (A + 1) blocks of 2 KB per head
    bp.flags = _lib.BWD_DS_WORKSPACE
    assert lib.axl_flash_bwd_workspace_bytes(ctypes.byref(bp)) == stats + 2 * 4 * 48 * 2048
    # ... of one of the two kv heads (2 query heads each) at a time: half of that; 2 or more heads is all of them
    bp.flags = _lib.BWD_DS_WORKSPACE | (1 << 8)   # AXL_BWD_DS_SLICE_KV_HEADS(1)
    assert lib.axl_flash_bwd_workspace_bytes(ctypes.byref(bp)) == stats + 2 * 2 * 48 * 2048
    bp.flags = _lib.BWD_DS_WORKSPACE | (2 << 8)
    assert lib.axl_flash_bwd_workspace_bytes(ctypes.byref(bp)) == stats + 2 * 4 * 48 * 2048
    bp.flags = 1 << 8                             # without AXL_BWD_DS_WORKSPACE the slice count means nothing
    assert lib.axl_flash_bwd_workspace_bytes(ctypes.byref(bp)) == stats
    bp.flags = _lib.BWD_DS_WORKSPACE
    # under a sliding window (or with segment ids): also which query tiles each 128-key block stored,
    # [B, S / 128] pairs of int32, rounded to 256 bytes
    bp.mask_kind = 2
    assert lib.axl_flash_bwd_workspace_bytes(ctypes.byref(bp)) == stats + 256 + 2 * 4 * 48 * 2048
    bp.segment_ids = 256
    assert lib.axl_flash_bwd_workspace_bytes(ctypes.byref(bp)) == stats + 256 + 256 + 2 * 4 * 48 * 2048
    bp.segment_ids = None
    bp.q_len = bp.kv_len = 384  # ... which at head_dim 128 needs 256-row blocks: the flag is ignored
    assert lib.axl_flash_bwd_workspace_bytes(ctypes.byref(bp)) == 2 * (2 * 4 * 384 * 4) + 240
    bp.q_len = bp.kv_len = 256
    bp.mask_kind = 0  # no mask: no dS workspace
    assert lib.axl_flash_bwd_workspace_bytes(ctypes.byref(bp)) == stats
    bp.mask_kind = 1
    bp.flags = 0
    # with segment ids: the table of id ranges per 32 rows, [B, T / 32] pairs of int32, rounded to 256 bytes
    bp.segment_ids = 256
    assert lib.axl_flash_bwd_workspace_bytes(ctypes.byref(bp)) == stats + 256
    bp.segment_ids = None
    assert lib.axl_flash_bwd(ctypes.byref(bp), None) == _lib.AXL_ERR_WORKSPACE
    # a pointer that is not 256-byte aligned is fine as long as the size covers the query (which
    # includes the rounding slack): the check that follows is the next one, not the workspace's
    bp.workspace, bp.workspace_bytes = 256 + 128, stats
    bp.d_logit_sink = 256
    assert lib.axl_flash_bwd(ctypes.byref(bp), None) == _lib.AXL_ERR_INVALID_ARGUMENT  # d_logit_sink without sink
    assert b"d_logit_sink" in lib.axl_last_error()
    bp.d_logit_sink = None
    bp.workspace = 256 + 8
    assert lib.axl_flash_bwd(ctypes.byref(bp), None) == _lib.AXL_ERR_WORKSPACE  # not 16-byte aligned
    bp.workspace, bp.workspace_bytes = 256, 16
    assert lib.axl_flash_bwd_phases(ctypes.byref(bp), 0, None) == _lib.AXL_ERR_INVALID_ARGUMENT
    # Paged decode geometry.
    dp = _lib.AxlPagedDecodeParams(q=256, k_pages=256, v_pages=256, page_tables=256, lengths=256, out=256, batch=2,
                                   num_q_heads=8, num_kv_heads=2, head_dim=128, num_pages=64, page_size=48,
                                   pages_per_seq=32, dtype=0, sliding_window=-1, softmax_scale=1.0, workspace=None,
                                   workspace_bytes=0)
    assert lib.axl_paged_decode(ctypes.byref(dp), None) == _lib.AXL_ERR_UNSUPPORTED  # 48 is not 16 * 2^k
    dp.page_size = 8
    assert lib.axl_paged_decode(ctypes.byref(dp), None) == _lib.AXL_ERR_UNSUPPORTED
    sizes = {}
    for page in (16, 32, 64, 128):  # what gpu_paged_attention.py:313-321 admits at its block of 128
        dp.page_size = page
        assert lib.axl_paged_decode(ctypes.byref(dp), None) == _lib.AXL_ERR_WORKSPACE
        sizes[page] = lib.axl_paged_decode_workspace_bytes(ctypes.byref(dp))
        assert sizes[page] > 0
    assert sizes[16] < sizes[32] < sizes[64]  # the split-K records follow the context the table can address
    dp.page_size = 16
    base = sizes[16]
    dp.num_q_heads = 64  # 32 query heads per kv head: two groups of 16, each with records of its own
    assert lib.axl_paged_decode(ctypes.byref(dp), None) == _lib.AXL_ERR_WORKSPACE
    assert lib.axl_paged_decode_workspace_bytes(ctypes.byref(dp)) > 2 * base
    dp.num_q_heads = 8
    dp.head_dim = 80   # between the compiled widths: served at 128
    assert lib.axl_paged_decode_workspace_bytes(ctypes.byref(dp)) == base
    dp.head_dim = 76   # not a multiple of 8
    assert lib.axl_paged_decode(ctypes.byref(dp), None) == _lib.AXL_ERR_UNSUPPORTED
    dp.head_dim = 128
    dp.bias = _lib.AxlDecodeBias(bias=256, batch_stride=0, head_stride=0, dtype=_lib.AXL_F16)
    assert lib.axl_paged_decode(ctypes.byref(dp), None) == _lib.AXL_ERR_UNSUPPORTED  # bias must be bf16 / fp32
    dp.bias.dtype = _lib.AXL_F32
    assert lib.axl_paged_decode_workspace_bytes(ctypes.byref(dp)) > base  # records padded to 16 head columns
    assert lib.axl_paged_decode(ctypes.byref(dp), None) == _lib.AXL_ERR_WORKSPACE


def test_ops_reject_mismatched_shapes_before_any_launch():
    """The tensor-level wrappers hand raw pointers to the kernels, so every extent that the kernels
    take from q / k alone is checked against the other tensors first.  CPU tensors suffice: the shape
    checks come before the device check and before the library is touched."""
    from axlearn_amd import ops

    bf = torch.bfloat16
    q = torch.zeros((2, 128, 4, 64), dtype=bf)
    k = torch.zeros((2, 128, 2, 64), dtype=bf)

    def raises(fn, *args, **kw):
        with pytest.raises(_lib.AxlError) as e:
            fn(*args, **kw)
        return e.value

    assert raises(ops.flash_fwd, q, k[:1], k[:1]).code == _lib.AXL_ERR_INVALID_ARGUMENT       # batch
    assert raises(ops.flash_fwd, q, k, k[:, :64]).code == _lib.AXL_ERR_INVALID_ARGUMENT       # v vs k
    assert raises(ops.flash_fwd, q, k[..., :32], k[..., :32]).code == _lib.AXL_ERR_INVALID_ARGUMENT  # head_dim
    assert raises(ops.flash_fwd, q[:, :, :3], k, k).code == _lib.AXL_ERR_INVALID_ARGUMENT     # 3 heads over 2
    assert raises(ops.flash_fwd, q, k.float(), k.float()).code == _lib.AXL_ERR_UNSUPPORTED    # dtypes differ
    seg = torch.zeros((2, 64), dtype=torch.int32)
    assert "segment_ids" in str(raises(ops.flash_fwd, q, k, k, segment_ids=seg))
    assert "q_pos_offsets" in str(raises(ops.flash_fwd, q, k, k, q_pos_offsets=torch.zeros(3, dtype=torch.int32)))
    # all shapes right: the next thing to fail is the device check
    assert "GPU" in str(raises(ops.flash_fwd, q, k, k, segment_ids=torch.zeros((2, 128), dtype=torch.int32)))

    lse = torch.zeros((2, 4, 128))
    assert "lse" in str(raises(ops.flash_bwd, q, k, k, q, lse[:, :2], q))
    assert "out" in str(raises(ops.flash_bwd, q, k, k, q[:, :64], lse, q))
    assert "d_out" in str(raises(ops.flash_bwd, q, k, k, q, lse, q[:1]))
    bufs = (torch.zeros_like(q), torch.zeros_like(k)[:, :64], torch.zeros_like(k), None)
    assert "buffers dk" in str(raises(ops.flash_bwd, q, k, k, q, lse, q, buffers=bufs))
    assert "GPU" in str(raises(ops.flash_bwd, q, k, k, q, lse, q))

    dq = torch.zeros((3, 8, 128), dtype=bf)
    pool = torch.zeros((2, 40, 16, 128), dtype=bf)
    tables = torch.zeros((3, 10), dtype=torch.int32)
    lengths = torch.zeros((3,), dtype=torch.int32)
    assert "page_tables" in str(raises(ops.paged_decode, dq, pool, pool, tables[:2], lengths))
    assert "lengths" in str(raises(ops.paged_decode, dq, pool, pool, tables, lengths[:2]))
    assert "v_pages" in str(raises(ops.paged_decode, dq, pool, pool[:, :39], tables, lengths))
    assert "head_dim" in str(raises(ops.paged_decode, dq[..., :64], pool, pool, tables, lengths))
    assert "int32" in str(raises(ops.paged_decode, dq, pool, pool, tables.long(), lengths))
    assert "out" in str(raises(ops.paged_decode, dq, pool, pool, tables, lengths, out=torch.zeros((3, 8, 64), dtype=bf)))
    assert "workspace" in str(raises(ops.paged_decode, dq, pool, pool, tables, lengths, workspace=torch.zeros(8)))
    assert "workspace_reused" in str(raises(ops.paged_decode, dq, pool, pool, tables, lengths, workspace_reused=True))
    assert "GPU" in str(raises(ops.paged_decode, dq, pool, pool, tables, lengths))

    kc = torch.zeros((3, 160, 2, 128), dtype=bf)
    assert "does not match" in str(raises(ops.decode, dq, kc[:2], kc[:2], lengths))
    assert "v" in str(raises(ops.decode, dq, kc, kc[:, :100], lengths))
    assert "lengths" in str(raises(ops.decode, dq, kc, kc, lengths[:1]))
    assert "GPU" in str(raises(ops.decode, dq, kc, kc, lengths))


def test_config_modifiers_rewrite_every_flash_config_in_a_tree():
    """FlashBlockSizeModifier / BackendOverrideModifier (layer.py:434-496): every FlashAttention config in
    the tree is rewritten; overrides are merged, falsy override values are not inserted."""
    import dataclasses

    from axlearn_amd.flash_attention.layer import BackendOverrideModifier, FlashAttention, FlashBlockSizeModifier

    @dataclasses.dataclass
    class Layer:
        attention: object
        other: int = 3

    @dataclasses.dataclass
    class Model:
        layers: list
        extra: dict

    a = FlashAttention.default_config()
    b = FlashAttention.default_config().set(backend_overrides=dict(save_residuals=True))
    c = FlashAttention.default_config()
    model = Model(layers=[Layer(a), Layer(b)], extra=dict(decoder=(Layer(c),), n=1))
    out = FlashBlockSizeModifier.default_config().set(tpu_block_size=1024, gpu_block_size=64).instantiate()(model)
    assert out is model
    for cfg in (a, b, c):
        assert (cfg.tpu_block_size, cfg.gpu_block_size) == (1024, 64)
    mod = BackendOverrideModifier.default_config().set(
        backend_overrides=dict(splash_block_q=2048, save_residuals=None)).instantiate()
    mod(model)
    assert a.backend_overrides == dict(splash_block_q=2048)
    assert b.backend_overrides == dict(save_residuals=True, splash_block_q=2048)   # merged, None not inserted
    BackendOverrideModifier.default_config().instantiate()(model)                  # no overrides: nothing changes
    assert c.backend_overrides == dict(splash_block_q=2048)


def test_layer_falls_back_when_no_kernel_supports_the_request():
    """`compute_attention` (layer.py:218-376): the bias reaches the dispatch cast to the query dtype
    (:253); when no kernel accepts the request (here: tensors on the CPU) the caller's standard attention
    runs with the ORIGINAL projections and the cast bias (:278-285); without one the call raises."""
    from axlearn_amd.flash_attention.layer import FlashAttention

    t = 128
    q = torch.zeros((1, t, 2, 64), dtype=torch.bfloat16)
    k = torch.zeros((1, t, 2, 64), dtype=torch.bfloat16)
    pos = dict(target_positions=torch.arange(t)[None], source_positions=torch.arange(t)[None])
    bias = ab.CompositeAttentionBias([ab.CausalAttentionBias(**pos)])
    assert bias.dtype is None
    layer = FlashAttention.default_config().instantiate()
    seen = {}

    def standard_attention(**kw):
        seen.update(kw)
        return "context", "probs"

    assert layer.compute_attention(q_proj=q, k_proj=k, v_proj=k, attention_logit_biases=bias,
                                   fallback=standard_attention) == ("context", "probs")
    assert seen["q_proj"] is q and seen["k_proj"] is k and seen["attention_logit_biases"].dtype == torch.bfloat16
    with pytest.raises(NotImplementedError):
        layer.compute_attention(q_proj=q, k_proj=k, v_proj=k, attention_logit_biases=bias)


def _device_asm(source, extra=()):
    """(assembly text, compiler remarks) of one kernel file, compiled as the Makefile compiles it."""
    import shutil
    import subprocess
    import tempfile

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "axlearn_amd", "csrc")
    with tempfile.TemporaryDirectory() as tmp:
        out_s = os.path.join(tmp, "kernel.s")
        cmd = [hipcc, "-O3", "-std=c++17", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", "-Wno-unused-value", "-Wno-unknown-attributes", "--cuda-device-only", "-S",
               "-Rpass-analysis=kernel-resource-usage", *extra, "-o", out_s, os.path.join(csrc, source)]
        out = subprocess.run(cmd, capture_output=True, text=True, cwd=csrc, timeout=900)
        assert out.returncode == 0, out.stderr[-2000:]
        return open(out_s).read(), out.stderr


def _assert_asm_mfma_distances(asm, pattern, want_kernels):
    """Every inline-assembly MFMA chain of the kernels whose name matches `pattern`: 12 wait states
    or two further MFMAs before anything else touches its registers, on every path; and no vector ALU
    write to a register an inline-assembly MFMA reads within the 8 wait states before it."""
    import isa_hazards  # tests/isa_hazards.py (pytest puts the test directory on sys.path)

    checked = 0
    for name, lines in isa_hazards.split_functions(asm).items():
        if not re.match(pattern, name):
            continue
        chains = sum(1 for l in lines if l.startswith("@v_mfma_"))
        bad = isa_hazards.check_function(lines)
        assert not bad, f"{name}: {len(bad)} hazards, first {bad[0]}"
        bad = isa_hazards.check_sources(lines)
        assert not bad, f"{name}: {len(bad)} operands written right before their MFMA, first {bad[0]}"
        checked += chains > 0
    assert checked == want_kernels, checked


def test_dkdv_kernel_keeps_its_vector_register_accumulators_in_place():
    """The plain dK/dV instantiations accumulate S and dP in vector registers through inline-assembly
    MFMAs, whose hazards the compiler does not see.  Three checks on what the compiler produced.
    Nothing spills: no scratch memory, and the AGPRs hold the dK / dV accumulators (head_dim of them)
    plus at most a few operand fragments that LDS reads fill and MFMAs consume directly.  Nothing is
    copied between the register files beyond setting the accumulators to zero and reading them out
    once (a build that moves chain registers through AGPRs shows more `v_accvgpr` instructions than
    that).  And on every path through every such kernel the first instruction that touches a chain's
    registers comes 12 wait states or two MFMAs after the chain's last MFMA."""
    import isa_hazards

    asm, remarks = _device_asm("flash_bwd_dkdv.hip")
    funcs = isa_hazards.split_functions(asm)
    seen = 0
    for block in remarks.split("Function Name: ")[1:]:
        name = block.split()[0]
        m = re.match(r"_ZN3axl21flash_bwd_dkdv_kernelINS_\d+Elem\w+ELi(\d+)ELb([01])ELi(\d+)ELb([01])EEE", name)
        if not m or m.group(3) != "0":  # other kernels; bias / dropout instantiations use the compiler's own form
            continue
        head_dim = int(m.group(1))
        agprs = int(re.search(r"AGPRs: (\d+)", block).group(1))
        scratch = int(re.search(r"ScratchSize \[bytes/lane\]: (\d+)", block).group(1))
        assert head_dim <= agprs <= head_dim + 16, f"{name}: {agprs} AGPRs"
        assert scratch == 0, f"{name}: scratch {scratch}"
        lines = [l.lstrip("@") for l in funcs[name]]
        reads = sum(l.startswith("v_accvgpr_read") for l in lines)
        writes = sum(l.startswith(("v_accvgpr_write", "v_accvgpr_mov")) for l in lines)
        assert reads == head_dim, f"{name}: {reads} AGPR reads"
        assert writes <= 2 * head_dim, f"{name}: {writes} AGPR writes"
        seen += 1
    assert seen == 16  # {bf16, f16} x {64, 128} x {plain, segment ids} x {recomputing, dS workspace}
    _assert_asm_mfma_distances(asm, r"_ZN3axl21flash_bwd_dkdv_kernel", 16)


def test_forward_kernel_keeps_the_distance_behind_its_assembly_mfma_chains():
    """The same for the forward's interior tiles, whose S^T chains of the next tile are inline-assembly
    MFMAs read by the softmax of the next step: the hazard distance on every path of the four
    instantiations that have such tiles ({bf16, f16} x {64, 128}, no bias / dropout).  (Any register
    the compiler spilled or copied right behind a chain would show up here as the first instruction
    that touches it.)"""
    asm, _ = _device_asm("flash_fwd.hip", extra=("-mllvm", "-amdgpu-mfma-vgpr-form"))
    _assert_asm_mfma_distances(asm, r"_ZN3axl16flash_fwd_kernel", 4)


def test_ffi_shim_and_jax_side_stay_in_step_with_the_abi():
    """csrc/ffi_shim.cc and flash_attention/jax_ffi.py only build and run under stand-ins here
    (test_jax_side.py: no jaxlib headers, no jax), so the pair is also checked from its text:
    every field the shim fills exists in the header's structure of that name (through the ctypes mirror,
    itself checked against the header), every handler binds as many operands, results and attributes -
    by name - as the JAX side passes to `jax.ffi.ffi_call`, and every registered target has a handler."""
    import ast

    pkg = os.path.join(ROOT, "axlearn_amd")
    shim = open(os.path.join(pkg, "csrc", "ffi_shim.cc")).read()
    shim_code = re.sub(r"//[^\n]*", "", shim)
    structs = {c.__name__: {f[0] for f in c._fields_} for c in (
        _lib.AxlFlashFwdParams, _lib.AxlFlashBwdParams, _lib.AxlDecodeParams, _lib.AxlPagedDecodeParams,
        _lib.AxlPageInsertParams, _lib.AxlAttnAux, _lib.AxlDecodeBias, _lib.AxlStrides)}
    # ---- fields filled through `T p{}` / `T* name` variables
    funcs = re.split(r"\nffi::Error (\w+)\(", shim_code)
    filled = 0
    for name, body in zip(funcs[1::2], funcs[2::2]):
        body = body[:body.find("\n}\n")]
        local = {v: t for t, v in re.findall(r"\b(Axl\w+)\s+(\w+)\{\}", body)}  # AxlDecodeParams p{}
        local.update({v: t for t, v in re.findall(r"\b(Axl\w+)\*\s+(\w+)\b", body)})  # AxlAttnAux* aux
        for var, typ in list(local.items()):
            if typ not in structs:
                continue
            for fld in re.findall(r"\b%s(?:\.|->)(\w+)\s*=[^=]" % re.escape(var), body):
                assert fld in structs[typ], f"{name}: {typ} has no field {fld}"
                filled += 1
    assert filled > 80
    # ---- bindings
    bound = {}
    for m in re.finditer(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\((\w+),\s*(\w+),(.*?)\);[ \t]*\n", shim_code, flags=re.S):
        target, func, bind = m.groups()
        assert re.search(r"\nffi::Error %s\(" % func, shim_code), func
        bound[target] = (len(re.findall(r"\.Arg<", bind)), len(re.findall(r"\.Ret<", bind)),
                         re.findall(r'\.Attr<\w+>\("(\w+)"\)', bind))
    # ---- the JAX side's calls
    tree = ast.parse(open(os.path.join(pkg, "flash_attention", "jax_ffi.py")).read())
    called = {}
    registered = None
    for node in ast.walk(tree):
        if isinstance(node, ast.Call) and isinstance(node.func, ast.Call) and ast.unparse(node.func.func).endswith("ffi_call"):
            inner = node.func
            results = inner.args[1]
            assert isinstance(results, (ast.Tuple, ast.List))
            called[inner.args[0].value] = (len(node.args), len(results.elts), [k.arg for k in node.keywords])
        if isinstance(node, ast.For) and "register_ffi_target" in ast.unparse(node):
            registered = [e.value for e in node.iter.elts]
    assert registered is not None and set(registered) == set(bound) == set(called)
    for target, (n_args, n_rets, attrs) in bound.items():
        assert called[target] == (n_args, n_rets, attrs), (target, called[target], (n_args, n_rets, attrs))
    # the version the shim and the binding were written against
    assert _lib.ABI_VERSION == int(re.search(r"#define AXL_ATTN_ABI_VERSION (\d+)",
                                             open(os.path.join(ROOT, "include", "axl_attn.h")).read()).group(1))
