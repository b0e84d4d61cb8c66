"""GPU test of axl_paged_decode_static, the entry point that allocates nothing: its split-K scratch is
a device array built into the library.  Called through the C ABI (ctypes) and compared with
axl_paged_decode, which takes the same kernels over a caller workspace: bit for bit with the fixed
work decomposition, to the bf16 bar of the decode tests (2e-2 max-abs or 1e-2 rel-L2 against the
oracle) otherwise.  Two calls in a row share the built-in buffer, the second on a smaller input, so
stale records, table entries and counters of the first call must not leak into the second."""

import ctypes

import pytest
import torch

from axlearn_amd import _lib
from oracle import ref_attention as ref

pytestmark = pytest.mark.gpu

STATIC_MAX_BYTES = 32 << 20  # AXL_PAGED_DECODE_STATIC_MAX_BYTES of include/axl_attn.h


def _params(q, kp, vp, tables, lengths, out, scale, flags, workspace=None):
    hkv, num_pages, page, d = kp.shape
    return _lib.AxlPagedDecodeParams(
        q=q.data_ptr(), k_pages=kp.data_ptr(), v_pages=vp.data_ptr(), page_tables=tables.data_ptr(),
        lengths=lengths.data_ptr(), out=out.data_ptr(), batch=q.shape[0], num_q_heads=q.shape[1],
        num_kv_heads=hkv, head_dim=d, num_pages=num_pages, page_size=page, pages_per_seq=tables.shape[1],
        dtype=_lib.dtype_code(q.dtype), sliding_window=-1, softmax_scale=scale,
        workspace=None if workspace is None else workspace.data_ptr(),
        workspace_bytes=0 if workspace is None else workspace.numel(), flags=flags)


def _case(seed, b, hq, hkv, d, pps, dev):
    q, kp, vp, tables, lengths = ref.paged_inputs(seed, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=1, max_len=16 * pps)
    want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=0.1, page_tables=tables)[:, 0]
    return [x.to(dev) for x in (q[:, 0].contiguous(), kp, vp, tables, lengths)], want


def test_static_scratch_decode_matches_workspace_decode():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    stream = _lib.current_stream_ptr()
    # the first call is the larger one; the second, smaller one runs over what the first left behind
    for seed, (b, hq, hkv, d, pps) in ((41, (9, 32, 8, 128, 96)), (43, (3, 8, 2, 128, 20))):
        (q, kp, vp, tables, lengths), want = _case(seed, b, hq, hkv, d, pps, dev)
        for flags in (_lib.DECODE_DETERMINISTIC, 0):
            out_ws, out_st = torch.zeros_like(q), torch.zeros_like(q)
            p = _params(q, kp, vp, tables, lengths, out_ws, 0.1, flags)
            need = int(lib.axl_paged_decode_workspace_bytes(ctypes.byref(p)))
            assert 0 < need <= STATIC_MAX_BYTES
            ws = torch.empty((need,), dtype=torch.uint8, device=dev)
            p = _params(q, kp, vp, tables, lengths, out_ws, 0.1, flags, ws)
            _lib.check(lib.axl_paged_decode(ctypes.byref(p), stream))
            before = torch.cuda.memory_allocated(dev)
            ps = _params(q, kp, vp, tables, lengths, out_st, 0.1, flags)  # no workspace
            _lib.check(lib.axl_paged_decode_static(ctypes.byref(ps), stream))
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated(dev) == before
            if flags & _lib.DECODE_DETERMINISTIC:
                assert torch.equal(out_st, out_ws), (seed, flags)
            else:
                assert ref.max_abs(out_st.cpu(), out_ws.cpu().float()) <= 2e-3, (seed, flags)
            got = out_st.cpu()
            assert ref.max_abs(got, want) <= 2e-2 or ref.rel_l2(got, want) <= 1e-2, (seed, flags)


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
