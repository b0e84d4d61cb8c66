"""GPU test of axl_paged_decode_static, the entry point that allocates nothing: its split-K scratch is
a device array built into the library.  Called through the C ABI (ctypes) and compared with
axl_paged_decode, which takes the same kernels over a caller workspace: bit for bit with the fixed
work decomposition, to the bf16 bar of the decode tests (1e-2 rel-L2 against the oracle: the
max-abs arm says nothing about outputs this small) otherwise.  Two calls in a row share the built-in buffer, the second on a smaller input, so
stale records, table entries and counters of the first call must not leak into the second."""

import ctypes
import gc

import pytest
import torch

from axlearn_amd import _lib
from oracle import ref_attention as ref

pytestmark = pytest.mark.gpu

STATIC_MAX_BYTES = 32 << 20  # AXL_PAGED_DECODE_STATIC_MAX_BYTES of include/axl_attn.h


def _params(q, kp, vp, tables, lengths, out, scale, flags, workspace=None, window=-1):
    hkv, num_pages, page, d = kp.shape
    return _lib.AxlPagedDecodeParams(
        q=q.data_ptr(), k_pages=kp.data_ptr(), v_pages=vp.data_ptr(), page_tables=tables.data_ptr(),
        lengths=lengths.data_ptr(), out=out.data_ptr(), batch=q.shape[0], num_q_heads=q.shape[1],
        num_kv_heads=hkv, head_dim=d, num_pages=num_pages, page_size=page, pages_per_seq=tables.shape[1],
        dtype=_lib.dtype_code(q.dtype), sliding_window=window, softmax_scale=scale,
        workspace=None if workspace is None else workspace.data_ptr(),
        workspace_bytes=0 if workspace is None else workspace.numel(), flags=flags)


def _case(seed, b, hq, hkv, d, pps, dev, dtype=torch.bfloat16, window=-1, empty=None):
    q, kp, vp, tables, lengths = ref.paged_inputs(seed, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=1, max_len=16 * pps,
                                                  dtype=dtype)
    if empty is not None:
        lengths[empty] = 0  # an empty context: all-zero output row, no record, no table entry
    want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=0.1, page_tables=tables,
                                sliding_window=None if window < 0 else window)[:, 0]
    return [x.to(dev) for x in (q[:, 0].contiguous(), kp, vp, tables, lengths)], want


def test_static_scratch_decode_matches_workspace_decode():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    stream = _lib.current_stream_ptr()
    resolved = False
    # the first call is the larger one; the later, smaller ones run over what it left behind in the
    # shared buffer: stale records, table entries and counters of other shapes and another dtype.  The
    # last two also take the fp32 kernels, a sliding window and a sequence of length 0.
    cases = (
        (41, (9, 32, 8, 128, 96), dict()),
        (43, (3, 8, 2, 128, 20), dict()),
        (47, (4, 8, 2, 64, 24), dict(dtype=torch.float32, window=37, empty=1)),
        (53, (2, 4, 4, 128, 12), dict(window=50, empty=0)),
    )
    for seed, (b, hq, hkv, d, pps), extra in cases:
        (q, kp, vp, tables, lengths), want = _case(seed, b, hq, hkv, d, pps, dev, **extra)
        window = extra.get("window", -1)
        for flags in (_lib.DECODE_DETERMINISTIC, 0):
            out_ws, out_st = torch.zeros_like(q), torch.full_like(q, float("nan"))
            p = _params(q, kp, vp, tables, lengths, out_ws, 0.1, flags, window=window)
            need = int(lib.axl_paged_decode_workspace_bytes(ctypes.byref(p)))
            assert 0 < need <= STATIC_MAX_BYTES
            ws = torch.empty((need,), dtype=torch.uint8, device=dev)
            p = _params(q, kp, vp, tables, lengths, out_ws, 0.1, flags, ws, window=window)
            _lib.check(lib.axl_paged_decode(ctypes.byref(p), stream))
            ps = _params(q, kp, vp, tables, lengths, out_st, 0.1, flags, window=window)  # no workspace
            if not resolved:  # the first call on a device looks the buffer's address up
                _lib.check(lib.axl_paged_decode_static(ctypes.byref(ps), stream))
                resolved = True
            torch.cuda.synchronize()
            # "allocates nothing": neither through torch's caching allocator nor behind its back (the
            # driver's count of free device memory, which a hipMalloc / hipFree inside the library moves).
            # Garbage that earlier tests left in reference cycles goes first: the collector would otherwise
            # be free to return its tensors in the middle of the measured call.
            gc.collect()
            before, free_before = torch.cuda.memory_allocated(dev), torch.cuda.mem_get_info(dev)[0]
            _lib.check(lib.axl_paged_decode_static(ctypes.byref(ps), stream))
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated(dev) == before
            assert torch.cuda.mem_get_info(dev)[0] == free_before
            if flags & _lib.DECODE_DETERMINISTIC or q.dtype == torch.float32:
                assert torch.equal(out_st, out_ws), (seed, flags)
            else:
                assert ref.max_abs(out_st.cpu(), out_ws.cpu().float()) <= 2e-3, (seed, flags)
            got, exp = out_st.cpu(), want
            if "empty" in extra:  # the kernels' o / (l + eps) gives zeros; the XLA oracle has no such row
                assert (got[extra["empty"]] == 0).all()
                live = [i for i in range(b) if i != extra["empty"]]
                got, exp = got[live], exp[live]
            if q.dtype == torch.float32:
                assert ref.max_abs(got, exp) <= 1e-5, (seed, flags)
            else:
                assert ref.rel_l2(got, exp) <= 1e-2, (seed, flags)


def test_static_scratch_decode_rejects_what_does_not_fit():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    b, hq, hkv, d, pps = 64, 32, 8, 128, 2048  # needs ~68 MB of scratch
    q = torch.zeros((b, hq, d), dtype=torch.bfloat16, device=dev)
    pool = torch.zeros((hkv, 64, 16, d), dtype=torch.bfloat16, device=dev)
    tables = torch.zeros((b, pps), dtype=torch.int32, device=dev)
    lengths = torch.ones((b,), dtype=torch.int32, device=dev)
    p = _params(q, pool, pool, tables, lengths, torch.empty_like(q), 0.1, 0)
    assert int(lib.axl_paged_decode_workspace_bytes(ctypes.byref(p))) > STATIC_MAX_BYTES
    assert lib.axl_paged_decode_static(ctypes.byref(p), _lib.current_stream_ptr()) == _lib.AXL_ERR_WORKSPACE
    assert b"built-in buffer" in lib.axl_last_error()
