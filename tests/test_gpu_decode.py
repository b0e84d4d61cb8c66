"""GPU parity tests of the paged and contiguous single-token decode kernels against the CPU oracle.

Shapes follow the reference's decoding tests (decoding_test.py:95-163, :187-269): (B, S, H, D) in
{(1,1024,32,64), (4,512,48,64), (2,1024,16,128), (1,4096,8,128)}, padding in {0, 111},
kv_head_factor in {1, 8}, window in {-1, 127}, page size 16.  Page-table and length masking are
checked bit-exactly (permutation invariance, poison) with the AXL_DECODE_DETERMINISTIC flag of the
call, which fixes the work decomposition; by default work is handed out dynamically and two calls
agree only up to the rounding of the fp32 partial sums, which is checked too.
"""

import contextlib
import functools

import numpy as np
import pytest
import torch

from axlearn_amd import attention_bias as ab
from axlearn_amd import ops
from axlearn_amd.flash_attention.hip_decoding import HipDecoding, HipPagedAttention
from axlearn_amd.flash_attention.utils import flash_attention_implementation
from axlearn_amd.kv_cache import KVCache, PagedKVCache
from oracle import brute
from oracle import ref_attention as ref

pytestmark = pytest.mark.gpu


@contextlib.contextmanager
def _deterministic():
    """Fixed work decomposition (every decode call inside carries the AXL_DECODE_DETERMINISTIC flag):
    the result does not depend on timing."""
    paged, contiguous = ops.paged_decode, ops.decode
    ops.paged_decode = functools.partial(paged, deterministic=True)
    ops.decode = functools.partial(contiguous, deterministic=True)
    try:
        yield
    finally:
        ops.paged_decode, ops.decode = paged, contiguous


def _ok(got, want):
    """The relative-L2 arm of the bf16 bar alone (as decoding_test.py:53-71 uses relative
    tolerances): a decode output over n keys has rms ~ sqrt(1/n), far below 2e-2 at long contexts,
    so the max-abs arm would pass a dropped page or a mis-merged split record."""
    return ref.rel_l2(got, want) <= 1e-2


@pytest.mark.parametrize("b,s,h,d", [(1, 1024, 32, 64), (4, 512, 48, 64), (2, 1024, 16, 128), (1, 4096, 8, 128)])
@pytest.mark.parametrize("padding", [0, 111])
@pytest.mark.parametrize("kv_head_factor", [1, 8])
@pytest.mark.parametrize("window", [-1, 127])
def test_paged_and_contiguous_decode_against_ref(b, s, h, d, padding, kv_head_factor, window):
    hkv = h // kv_head_factor
    pps = s // 16
    q, kp, vp, tables, _ = ref.paged_inputs(3, batch=b, num_heads=h, num_kv_heads=hkv, head_dim=d, page_size=16,
                                            pages_per_seq=pps, min_len=1, max_len=s)
    lengths = torch.full((b,), s - padding, dtype=torch.int32)
    scale = d ** -0.5
    want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=scale, page_tables=tables,
                                sliding_window=None if window < 0 else window)[:, 0]
    got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                           softmax_scale=scale, sliding_window=window)
    assert _ok(got.cpu(), want), (ref.max_abs(got.cpu(), want), ref.rel_l2(got.cpu(), want))
    kk, vv = ref.reconstruct_kv(tables, kp), ref.reconstruct_kv(tables, vp)
    got2 = ops.decode(q[:, 0].cuda(), kk.cuda(), vv.cuda(), lengths.cuda(), softmax_scale=scale, sliding_window=window)
    assert _ok(got2.cpu(), want)
    # Same arithmetic on the same tokens in the same order: paged and contiguous agree bit for bit.
    with _deterministic():
        det = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                               softmax_scale=scale, sliding_window=window)
        det2 = ops.decode(q[:, 0].cuda(), kk.cuda(), vv.cuda(), lengths.cuda(), softmax_scale=scale,
                          sliding_window=window)
    assert _ok(det.cpu(), want) and torch.equal(det, det2)
    assert ref.max_abs(got.cpu(), det.cpu().float()) <= 2e-3


@pytest.mark.parametrize("b,s,h,hkv", [
    (1, 1024, 8, 8),     # 8 rows of 64 pages: 8-page blocks, dealt by workgroup index
    (4, 2048, 8, 8),     # 32 rows: exactly as many 8-page blocks as workgroup slots
    (5, 2048, 8, 8),     # 40 rows: 12-page blocks, 11 per row
    (3, 1040, 32, 2),    # a last block shorter than the others
    (32, 1024, 8, 8),    # 256 rows of two 32-page blocks: not shortened, still one block per workgroup
    (33, 1024, 8, 8),    # one row more: drawn from the counter again
])
def test_small_calls_take_short_blocks(b, s, h, hkv):
    """Calls with fewer 32-page blocks than the split kernel has workgroup slots (512 on an MI355X) take
    shorter blocks and, where the shapes bound the blocks by the workgroups, are dealt by workgroup index
    without the work counter: ragged lengths, with and without a window, against the oracle, on a
    workspace full of NaN bit patterns (a counter that was read, or a record that was not written,
    shows), and bit-identical between the paged and the contiguous form under the fixed decomposition."""
    d = 128
    pps = (s + 15) // 16
    q, kp, vp, tables, lengths = ref.paged_inputs(21, batch=b, num_heads=h, num_kv_heads=hkv, head_dim=d, page_size=16,
                                                   pages_per_seq=pps, min_len=1, max_len=s)
    lengths[0] = s   # the longest context takes every block of its row
    scale = d ** -0.5
    args = (q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda())
    need = ops.paged_decode_workspace_bytes(b, h, hkv, d, pps)
    for window in (-1, 200):
        want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=scale, page_tables=tables,
                                    sliding_window=None if window < 0 else window)[:, 0]
        ws = torch.full((need,), 0xFF, dtype=torch.uint8, device="cuda")
        got = ops.paged_decode(*args, softmax_scale=scale, sliding_window=window, workspace=ws)
        assert torch.isfinite(got.float()).all() and _ok(got.cpu(), want), (window, ref.rel_l2(got.cpu(), want))
        kk, vv = ref.reconstruct_kv(tables, kp), ref.reconstruct_kv(tables, vp)
        with _deterministic():
            ws.fill_(0xFF)
            det_p = ops.paged_decode(*args, softmax_scale=scale, sliding_window=window, workspace=ws)
            det_c = ops.decode(args[0], kk[:, :s].contiguous().cuda(), vv[:, :s].contiguous().cuda(), args[4],
                               softmax_scale=scale, sliding_window=window)
        assert _ok(det_p.cpu(), want) and torch.equal(det_p, det_c)


def test_ragged_lengths_and_brute_force():
    b, hq, hkv, d, pps = 5, 8, 2, 128, 24
    q, kp, vp, tables, lengths = ref.paged_inputs(7, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=1, max_len=16 * pps)
    lengths[0], lengths[1], lengths[2] = 1, 16, 17  # single token, exactly one page, one page + 1
    scale = 0.11
    want = brute.paged_decode(q[:, 0].float().numpy(), kp.float().numpy(), vp.float().numpy(), tables.numpy(),
                              lengths.numpy(), scale=scale)
    got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(), softmax_scale=scale)
    assert _ok(got.cpu(), torch.from_numpy(want))
    # A single live token: the output is that token's V row exactly.
    first = int(tables[0, 0])
    g = hq // hkv
    for hh in range(hq):
        assert torch.equal(got[0, hh].cpu(), vp[hh // g, first, 0])


def test_page_table_permutation_invariance_bit_exact():
    b, hq, hkv, d, pps = 4, 8, 2, 128, 40
    q, kp, vp, tables, lengths = ref.paged_inputs(9, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=30, max_len=16 * pps)
    with _deterministic():
        base = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(), softmax_scale=0.09)
    total = b * pps
    perm = torch.from_numpy(np.random.default_rng(1).permutation(total))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(total)
    tables2 = inv[tables.long()].to(torch.int32)
    with _deterministic():
        again = ops.paged_decode(q[:, 0].cuda(), kp[:, perm].contiguous().cuda(), vp[:, perm].contiguous().cuda(),
                                 tables2.cuda(), lengths.cuda(), softmax_scale=0.09)
    assert torch.equal(base, again)
    dyn = ops.paged_decode(q[:, 0].cuda(), kp[:, perm].contiguous().cuda(), vp[:, perm].contiguous().cuda(),
                           tables2.cuda(), lengths.cuda(), softmax_scale=0.09)
    assert ref.max_abs(dyn.cpu(), base.cpu().float()) <= 2e-3


def test_length_masking_poison_and_oob_pages():
    b, hq, hkv, d, pps = 3, 4, 1, 128, 20
    q, kp, vp, tables, lengths = ref.paged_inputs(13, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=10, max_len=16 * pps - 40)
    qc, tc, lc = q[:, 0].cuda(), tables.cuda(), lengths.cuda()
    with _deterministic():
        base = ops.paged_decode(qc, kp.cuda(), vp.cuda(), tc, lc, softmax_scale=0.1)
    kpo, vpo = kp.clone(), vp.clone()
    for bi in range(b):
        n = int(lengths[bi])
        for j in range(n, 16 * pps):  # every token at or beyond the length, incl. whole unused pages
            pg = int(tables[bi, j // 16])
            kpo[:, pg, j % 16] = float("nan")
            vpo[:, pg, j % 16] = float("nan")
    with _deterministic():
        poisoned = ops.paged_decode(qc, kpo.cuda(), vpo.cuda(), tc, lc, softmax_scale=0.1)
    assert torch.equal(base, poisoned) and torch.isfinite(poisoned.float()).all()
    dyn = ops.paged_decode(qc, kpo.cuda(), vpo.cuda(), tc, lc, softmax_scale=0.1)
    assert torch.isfinite(dyn.float()).all() and ref.max_abs(dyn.cpu(), base.cpu().float()) <= 2e-3
    # Out-of-pool page index inside the live range reads as zeros and a negative one counts from
    # the end of the pool, like reconstruct_kv.
    t2 = tables.clone()
    t2[0, 0] = b * pps + 5
    t2[1, 0] = -3
    lengths2 = torch.maximum(lengths, torch.tensor(40, dtype=torch.int32))
    want = ref.reference_decode(q, kp, vp, lengths2, softmax_scale=0.1, page_tables=t2)[:, 0]
    got = ops.paged_decode(qc, kp.cuda(), vp.cuda(), t2.cuda(), lengths2.cuda(), softmax_scale=0.1)
    assert _ok(got.cpu(), want)


def test_decode_equals_last_row_of_prefill():
    b, hq, hkv, d, s = 2, 8, 2, 128, 512
    k = ref.normal_tensor(1, (b, s, hkv, d), torch.bfloat16).cuda()
    v = ref.normal_tensor(2, (b, s, hkv, d), torch.bfloat16).cuda()
    q = ref.normal_tensor(0, (b, s, hq, d), torch.bfloat16).cuda()
    full, _ = ops.flash_fwd(q, k, v, softmax_scale=d ** -0.5, mask_kind=ops.MASK_CAUSAL)
    lengths = torch.full((b,), s, dtype=torch.int32).cuda()
    dec = ops.decode(q[:, -1].contiguous(), k, v, lengths, softmax_scale=d ** -0.5)
    assert _ok(dec.cpu(), full[:, -1].cpu())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_dispatch_decode_end_to_end(dtype):
    b, hq, hkv, d, pps = 4, 16, 2, 64, 32
    q, kp, vp, tables, lengths = ref.paged_inputs(21, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=5, max_len=16 * pps,
                                                  dtype=dtype)

    def _ok(got, want):  # the bars of the three dtypes
        if dtype == torch.float32:
            return got.dtype == dtype and ref.max_abs(got, want) <= 1e-5
        f = 1.0 if dtype == torch.bfloat16 else 0.125
        return got.dtype == dtype and ref.rel_l2(got, want) <= 1e-2 * f

    tp = (lengths.long() - 1)[:, None].cuda()
    sp = torch.arange(16 * pps)[None].cuda()
    scale = d ** -0.5
    bias = ab.CompositeAttentionBias([ab.CausalAttentionBias(target_positions=tp, source_positions=sp)])
    args = dict(query=q.cuda(), key=kp.cuda(), value=vp.cuda(), bias=bias)
    impl = flash_attention_implementation("gpu", **args, softmax_scale=scale, kv_cache_type=PagedKVCache,
                                          page_tables=tables.cuda())
    assert impl is not None and isinstance(impl.fn, HipPagedAttention)
    got = impl.fn(dict(**args, page_tables=tables.cuda()))
    want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=scale, page_tables=tables)
    assert got.shape == (b, 1, hq, d) and _ok(got.cpu(), want)
    # Contiguous cache through the non-paged table; sliding-window bias.
    kk, vv = ref.reconstruct_kv(tables, kp).cuda(), ref.reconstruct_kv(tables, vp).cuda()
    wbias = ab.CompositeAttentionBias([ab.SlidingWindowAttentionBias(
        ab.sliding_window_causal_mask(50), sliding_window_size=50, target_positions=tp, source_positions=sp)])
    impl = flash_attention_implementation("gpu", query=q.cuda(), key=kk, value=vv, bias=wbias, softmax_scale=scale,
                                          kv_cache_type=KVCache)
    assert impl is not None and isinstance(impl.fn, HipDecoding)
    got = impl.fn(dict(query=q.cuda(), key=kk, value=vv, bias=wbias))
    want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=scale, page_tables=tables, sliding_window=50)
    assert _ok(got.cpu(), want)
    # Multi-token query with a KV cache is not a decode step: the decode kernel declines and the
    # prefill kernel does not take cached calls either -> None.
    q2 = torch.zeros(b, 2, hq, d, dtype=dtype, device="cuda")
    assert flash_attention_implementation("gpu", query=q2, key=kk, value=vv, bias=wbias, kv_cache_type=KVCache) is None


def test_decode_replays_from_a_captured_graph():
    """The decode call enqueues kernels only (no memsets, no allocation inside the library, no
    synchronisation), so it can be captured into a graph.  Every replay, with eager work between the
    replays, must equal the eager result bit for bit (fixed decomposition)."""
    b, hq, hkv, d, pps = 5, 16, 4, 128, 40
    q, kp, vp, tables, lengths = ref.paged_inputs(31, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=3, max_len=16 * pps)
    qc, kc, vc, tc, lc = q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda()
    kk, vv = ref.reconstruct_kv(tables, kp).cuda(), ref.reconstruct_kv(tables, vp).cuda()
    with _deterministic():
        ws = torch.empty((ops.paged_decode_workspace_bytes(b, hq, hkv, d, pps) + 16,), dtype=torch.uint8, device="cuda")
        ws2 = torch.empty_like(ws)
        out_g, out_g2 = torch.empty_like(qc), torch.empty_like(qc)
        eager = ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):  # warm-up outside the capture
            ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1, workspace=ws, out=out_g)
            ops.decode(qc, kk, vv, lc, softmax_scale=0.1, workspace=ws2, out=out_g2)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1, workspace=ws, out=out_g)
            ops.decode(qc, kk, vv, lc, softmax_scale=0.1, workspace=ws2, out=out_g2)
        for rep in range(3):
            out_g.zero_()
            out_g2.zero_()
            ws.random_(0, 255)  # stale records and counters must not matter
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out_g, eager) and torch.equal(out_g2, eager), rep
            # eager work of the same kind between the replays
            again = ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1)
            assert torch.equal(again, eager)
            # new inputs in the captured buffers are picked up by the next replay
            lc.copy_(torch.clamp(lengths + 7 * (rep + 1), max=16 * pps).cuda())
            eager = ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("window", [-1, 40])
def test_empty_and_out_of_range_lengths(dtype, window):
    """A sequence without a visible key gets zeros (the reference's combine divides by l + eps,
    gpu_decoding.py:282, gpu_paged_attention.py:291-293); lengths beyond the capacity are clamped to
    it; negative lengths count as 0.  The other rows are unaffected and finite."""
    b, hq, hkv, d, pps = 6, 8, 2, 128, 12
    q, kp, vp, tables, lengths = ref.paged_inputs(17, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=5, max_len=16 * pps,
                                                  dtype=dtype)
    cap = 16 * pps
    lengths[1], lengths[3], lengths[4] = 0, cap + 1000, -7
    clamped = lengths.clamp(0, cap)
    live = [i for i in range(b) if int(clamped[i]) > 0]
    want = ref.reference_decode(q[live], kp, vp, clamped[live], softmax_scale=0.1, page_tables=tables[live],
                                sliding_window=None if window < 0 else window)[:, 0]
    kk, vv = ref.reconstruct_kv(tables, kp), ref.reconstruct_kv(tables, vp)
    tol = dict(atol=1e-5) if dtype == torch.float32 else None
    for det in (False, True):
        got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(), softmax_scale=0.1,
                               sliding_window=window, deterministic=det).cpu()
        got2 = ops.decode(q[:, 0].cuda(), kk.cuda(), vv.cuda(), lengths.cuda(), softmax_scale=0.1,
                          sliding_window=window, deterministic=det).cpu()
        for out in (got, got2):
            assert torch.isfinite(out.float()).all()
            assert (out[1] == 0).all() and (out[4] == 0).all()
            if tol:
                assert ref.max_abs(out[live], want) <= 1e-5
            else:
                assert _ok(out[live], want), (ref.max_abs(out[live], want), ref.rel_l2(out[live], want))
    # every sequence empty
    zero = torch.zeros((b,), dtype=torch.int32)
    out = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), zero.cuda(), softmax_scale=0.1,
                           sliding_window=window)
    assert (out == 0).all()


def test_reused_workspace_skips_the_counter_reset():
    """With AXL_DECODE_WORKSPACE_REUSED the call relies on the counter its predecessor left at zero:
    eager calls of different shapes on one workspace and graph replays all equal the plain call."""
    b, hq, hkv, d, pps = 7, 16, 4, 128, 48
    q, kp, vp, tables, lengths = ref.paged_inputs(33, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=3, max_len=16 * pps)
    qc, kc, vc, tc, lc = q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda()
    kk, vv = ref.reconstruct_kv(tables, kp).cuda(), ref.reconstruct_kv(tables, vp).cuda()
    want = ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1, deterministic=True)
    ws = torch.empty((ops.paged_decode_workspace_bytes(b, hq, hkv, d, pps) + 64,), dtype=torch.uint8, device="cuda")
    ws.random_(0, 255)
    first = ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1, deterministic=True, workspace=ws)  # resets
    assert torch.equal(first, want)
    for rep in range(3):
        again = ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1, deterministic=True, workspace=ws,
                                 workspace_reused=True)
        assert torch.equal(again, want), rep
        # another shape (fewer sequences, contiguous cache, dynamic hand-out) in between
        other = ops.decode(qc[:3], kk[:3], vv[:3], lc[:3], softmax_scale=0.1, workspace=ws, workspace_reused=True)
        assert ref.max_abs(other.cpu(), want[:3].cpu().float()) <= 2e-3
        dyn = ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1, workspace=ws, workspace_reused=True)
        assert ref.max_abs(dyn.cpu(), want.cpu().float()) <= 2e-3
    out_g = torch.empty_like(qc)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1, deterministic=True, workspace=ws, out=out_g,
                         workspace_reused=True)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1, deterministic=True, workspace=ws, out=out_g,
                         workspace_reused=True)
    for rep in range(3):
        out_g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, want), rep
        eager = ops.paged_decode(qc, kc, vc, tc, lc, softmax_scale=0.1, deterministic=True)
        assert torch.equal(eager, want)


def test_baseline_c4_full_size():
    """BASELINE config 4 at full size; the oracle checks a sample of sequences (incl. the shortest
    and the longest), the rest is covered by permutation invariance at full size."""
    B, Hq, Hkv, D, pps = 64, 32, 8, 128, 2048
    P = B * pps
    dev = "cuda"
    gen = torch.Generator(device=dev).manual_seed(1)
    kp = torch.empty((Hkv, P, 16, D), device=dev, dtype=torch.bfloat16)
    vp = torch.empty((Hkv, P, 16, D), device=dev, dtype=torch.bfloat16)
    for h in range(Hkv):
        kp[h] = torch.randn((P, 16, D), device=dev, generator=gen).to(torch.bfloat16)
        vp[h] = torch.randn((P, 16, D), device=dev, generator=gen).to(torch.bfloat16)
    q = torch.randn((B, Hq, D), device=dev, generator=gen).to(torch.bfloat16)
    lengths = torch.from_numpy(np.random.default_rng(5).integers(512, 32769, size=B).astype(np.int32))
    tables = torch.from_numpy(np.random.default_rng(6).permutation(P).astype(np.int32)).reshape(B, pps)
    scale = D ** -0.5
    out = ops.paged_decode(q, kp, vp, tables.to(dev), lengths.to(dev), softmax_scale=scale)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    sample = sorted({0, 17, int(lengths.argmin()), int(lengths.argmax())})
    for bi in sample:
        n_pages = (int(lengths[bi]) + 15) // 16
        idx = tables[bi, :n_pages].long().to(dev)
        k_seq = kp[:, idx].cpu()  # [Hkv, n_pages, 16, D]
        v_seq = vp[:, idx].cpu()
        local = torch.arange(n_pages, dtype=torch.int32)[None]
        want = ref.reference_decode(q[bi:bi + 1].cpu().unsqueeze(1), k_seq, v_seq, lengths[bi:bi + 1],
                                    softmax_scale=scale, page_tables=local)[:, 0]
        assert _ok(out[bi:bi + 1].cpu(), want), bi
    with _deterministic():
        det = ops.paged_decode(q, kp, vp, tables.to(dev), lengths.to(dev), softmax_scale=scale)
    assert ref.max_abs(det.cpu(), out.cpu().float()) <= 2e-3
    # Swap the physical location of two sequences' pages (pool-level permutation on a slice).
    tables2 = tables.clone()
    a, c = tables2[3].clone(), tables2[40].clone()
    kp2, vp2 = kp, vp  # in place: swap page contents and table entries
    ka, kc = kp2[:, a.long().to(dev)].clone(), kp2[:, c.long().to(dev)].clone()
    va, vc = vp2[:, a.long().to(dev)].clone(), vp2[:, c.long().to(dev)].clone()
    kp2[:, a.long().to(dev)], kp2[:, c.long().to(dev)] = kc, ka
    vp2[:, a.long().to(dev)], vp2[:, c.long().to(dev)] = vc, va
    tables2[3], tables2[40] = c, a
    out2 = ops.paged_decode(q, kp2, vp2, tables2.to(dev), lengths.to(dev), softmax_scale=scale)
    # Work is handed to workgroups dynamically, so the fp32 partial sums may be grouped differently
    # from call to call: equal up to the rounding of the fp32 merge, far inside the bf16 tolerance.
    assert ref.max_abs(out2.cpu(), out.cpu().float()) <= 2e-3
    with _deterministic():
        det2 = ops.paged_decode(q, kp2, vp2, tables2.to(dev), lengths.to(dev), softmax_scale=scale)
    assert torch.equal(det, det2)
    # The same pools read as 64-token pages (four adjacent 16-token pages each) under a table of their
    # own: the oracle checks the sampled sequences again, and the result does not depend on which page
    # size the same tokens are addressed through (fixed decomposition: bit for bit).
    kp64, vp64 = kp2.view(Hkv, P // 4, 64, D), vp2.view(Hkv, P // 4, 64, D)
    tables64 = torch.from_numpy(np.random.default_rng(8).permutation(P // 4).astype(np.int32)).reshape(B, pps // 4)
    out64 = ops.paged_decode(q, kp64, vp64, tables64.to(dev), lengths.to(dev), softmax_scale=scale)
    for bi in sample:
        n_pages = (int(lengths[bi]) + 63) // 64
        idx = tables64[bi, :n_pages].long().to(dev)
        local = torch.arange(n_pages, dtype=torch.int32)[None]
        want = ref.reference_decode(q[bi:bi + 1].cpu().unsqueeze(1), kp64[:, idx].cpu(), vp64[:, idx].cpu(),
                                    lengths[bi:bi + 1], softmax_scale=scale, page_tables=local)[:, 0]
        assert _ok(out64[bi:bi + 1].cpu(), want), bi
    # ... 16-token tables that spell out the same physical tokens
    tables16 = (4 * tables64[:, :, None] + torch.arange(4, dtype=torch.int32)[None, None, :]).reshape(B, pps)
    with _deterministic():
        a64 = ops.paged_decode(q, kp64, vp64, tables64.to(dev), lengths.to(dev), softmax_scale=scale)
        a16 = ops.paged_decode(q, kp2, vp2, tables16.to(dev), lengths.to(dev), softmax_scale=scale)
    assert torch.equal(a64, a16)


def test_wide_groups_and_batch_slices():
    """16 query heads per kv head, and a batch larger than one launch's share (512 sequences)."""
    for (b, hq, hkv, d, pps) in [(3, 32, 2, 128, 12), (2, 16, 1, 64, 9), (700, 4, 2, 64, 3)]:
        q, kp, vp, tables, lengths = ref.paged_inputs(31, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                      page_size=16, pages_per_seq=pps, min_len=1, max_len=16 * pps)
        want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=0.11, page_tables=tables)[:, 0]
        got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(), softmax_scale=0.11)
        assert _ok(got.cpu(), want), (b, hq, hkv, d, ref.max_abs(got.cpu(), want))
        kk, vv = ref.reconstruct_kv(tables, kp), ref.reconstruct_kv(tables, vp)
        got2 = ops.decode(q[:, 0].cuda(), kk.cuda(), vv.cuda(), lengths.cuda(), softmax_scale=0.11)
        assert _ok(got2.cpu(), want), (b, hq, hkv, d)


@pytest.mark.parametrize("b,s,h,hkv,d,padding,window", [
    (2, 1024, 16, 2, 128, 111, -1),
    (4, 512, 48, 48, 64, 0, 127),
    (3, 2048, 32, 8, 128, 37, -1),
])
def test_float16_decode_against_ref(b, s, h, hkv, d, padding, window):
    """float16 (the reference's decode tests run float32 and float16 on GPU, decoding_test.py:33):
    same kernels with the f16 matrix instructions; the bar is 8x tighter than bf16's, as the
    mantissa is."""
    pps = s // 16
    q, kp, vp, tables, _ = ref.paged_inputs(11, batch=b, num_heads=h, num_kv_heads=hkv, head_dim=d, page_size=16,
                                            pages_per_seq=pps, min_len=1, max_len=s, dtype=torch.float16)
    lengths = torch.full((b,), s - padding, dtype=torch.int32)
    lengths[0] = max(1, s // 3)
    scale = d ** -0.5
    want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=scale, page_tables=tables,
                                sliding_window=None if window < 0 else window)[:, 0]

    def ok(got):
        return got.dtype == torch.float16 and ref.rel_l2(got.cpu(), want) <= 1.25e-3

    got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                           softmax_scale=scale, sliding_window=window)
    assert ok(got), (ref.max_abs(got.cpu(), want), ref.rel_l2(got.cpu(), want))
    kk, vv = ref.reconstruct_kv(tables, kp), ref.reconstruct_kv(tables, vp)
    got2 = ops.decode(q[:, 0].cuda(), kk.cuda(), vv.cuda(), lengths.cuda(), softmax_scale=scale, sliding_window=window)
    assert ok(got2), (ref.max_abs(got2.cpu(), want), ref.rel_l2(got2.cpu(), want))
    with _deterministic():
        det = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                               softmax_scale=scale, sliding_window=window)
        det2 = ops.decode(q[:, 0].cuda(), kk.cuda(), vv.cuda(), lengths.cuda(), softmax_scale=scale,
                          sliding_window=window)
    assert ok(det) and torch.equal(det, det2)


@pytest.mark.parametrize("b,s,h,hkv,d,padding,window", [
    (1, 1024, 32, 32, 64, 0, -1),     # shapes of decoding_test.py:95-163
    (4, 512, 48, 6, 64, 111, -1),
    (2, 1024, 16, 2, 128, 111, 127),
    (1, 4096, 8, 1, 128, 0, -1),
    (3, 640, 12, 4, 128, 5, 33),
])
def test_float32_decode_against_ref(b, s, h, hkv, d, padding, window):
    """float32 (the reference's decode tests run float32 and float16 on GPU, decoding_test.py:33)
    at the fp32 bar; paged and contiguous agree bit for bit (same arithmetic, fixed decomposition),
    and a poisoned tail beyond the length changes nothing."""
    pps = s // 16
    q, kp, vp, tables, _ = ref.paged_inputs(13, batch=b, num_heads=h, num_kv_heads=hkv, head_dim=d, page_size=16,
                                            pages_per_seq=pps, min_len=1, max_len=s, dtype=torch.float32)
    lengths = torch.full((b,), s - padding, dtype=torch.int32)
    lengths[0] = max(1, s // 3 + 1)
    scale = d ** -0.5
    want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=scale, page_tables=tables,
                                sliding_window=None if window < 0 else window)[:, 0]
    got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                           softmax_scale=scale, sliding_window=window)
    assert got.dtype == torch.float32 and ref.max_abs(got.cpu(), want) <= 1e-5, ref.max_abs(got.cpu(), want)
    kk, vv = ref.reconstruct_kv(tables, kp), ref.reconstruct_kv(tables, vp)
    for bi in range(b):  # rows at and beyond the length are never read into the result
        kk[bi, int(lengths[bi]):] = float("nan")
        vv[bi, int(lengths[bi]):] = float("nan")
    got2 = ops.decode(q[:, 0].cuda(), kk.cuda(), vv.cuda(), lengths.cuda(), softmax_scale=scale, sliding_window=window)
    assert torch.equal(got2, got)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("page_size,d", [(16, 128), (8, 64), (32, 128)])
def test_paged_kv_insert_bit_exact(dtype, page_size, d):
    """Page insert against the oracle, bit for bit: live rows, padding page, positions and pages out of
    range, one position broadcast over the batch; then paged decode sees the new token."""
    from axlearn_amd import kv_cache as kvc

    hkv, b, pps = 4, 9, 6
    total = b * pps + 1
    g = torch.Generator().manual_seed(5)
    kp = torch.randn((hkv, total, page_size, d), generator=g).to(dtype)
    vp = torch.randn((hkv, total, page_size, d), generator=g).to(dtype)
    perm = torch.from_numpy(np.random.default_rng(3).permutation(total - 1).astype(np.int32) + 1)
    tables = perm[: b * pps].reshape(b, pps).clone()
    pos = torch.from_numpy(np.random.default_rng(4).integers(0, page_size * pps, size=(b, 1)).astype(np.int32))
    tables[1, int(pos[1, 0]) // page_size] = 0            # padding page: never written
    pos[2, 0] = page_size * pps                           # position past the table
    pos[3, 0] = -3                                        # negative position
    tables[4, int(pos[4, 0]) // page_size] = total + 5    # page outside the pool
    k_new = torch.randn((b, 1, hkv, d), generator=g)
    v_new = torch.randn((b, 1, hkv, d), generator=g)
    want_k = ref.scatter_update_pages(kp, k_new.to(dtype).permute(2, 0, 1, 3), tables, pos)
    want_v = ref.scatter_update_pages(vp, v_new.to(dtype).permute(2, 0, 1, 3), tables, pos)
    kd, vd = kp.cuda(), vp.cuda()
    kvc.paged_extend_step(kd, vd, tables.cuda(), k_proj=k_new.cuda(), v_proj=v_new.cuda(), key_positions=pos.cuda())
    assert torch.equal(kd.cpu(), want_k) and torch.equal(vd.cpu(), want_v)
    assert int((want_k != kp).any(dim=-1).sum()) == hkv * (b - 4)
    # The reference's kernel-level entry point: one pool, projections laid out [heads, batch, 1, D].
    kd2 = kp.cuda()
    out = kvc.scatter_update_pages_kernel(kv_pages=kd2, kv_proj=k_new.to(dtype).permute(2, 0, 1, 3).contiguous().cuda(),
                                          page_indices=tables.cuda(), key_positions=pos.cuda())
    assert out is kd2 and torch.equal(kd2.cpu(), want_k)
    # One position for the whole batch.
    kd3 = kp.cuda()
    one = torch.tensor([[page_size + 1]], dtype=torch.int32)
    ops.paged_kv_insert(kd3, None, k_new[:, 0].to(dtype).cuda(), None, tables.cuda(), one.reshape(-1).cuda())
    assert torch.equal(kd3.cpu(), ref.scatter_update_pages(kp, k_new.to(dtype).permute(2, 0, 1, 3), tables, one))
    if dtype == torch.bfloat16 and page_size == 16:
        lengths = (pos[:, 0] + 1).clamp(min=1, max=page_size * pps).to(torch.int32)
        q = torch.randn((b, 1, hkv * 2, d), generator=g).to(dtype)
        want = ref.reference_decode(q, want_k, want_v, lengths, softmax_scale=0.1, page_tables=tables)[:, 0]
        got = ops.paged_decode(q[:, 0].cuda(), kd, vd, tables.cuda(), lengths.cuda(), softmax_scale=0.1)
        assert _ok(got.cpu(), want)


def test_decode_edge_lengths_and_random_shapes():
    """Lengths of 1, of exactly one page, of a whole number of pages and of the full table; window 0
    (the query sees only itself); then a seeded sweep of random shapes against the oracle."""
    hq, hkv, d, pps = 8, 2, 128, 7
    lengths = torch.tensor([1, 16, 17, 32, 111, 112], dtype=torch.int32)
    b = lengths.numel()
    q, kp, vp, tables, _ = ref.paged_inputs(41, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d, page_size=16,
                                            pages_per_seq=pps, min_len=1, max_len=16 * pps)
    for window in (-1, 0, 5):
        want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=0.2, page_tables=tables,
                                    sliding_window=None if window < 0 else window)[:, 0]
        got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                               softmax_scale=0.2, sliding_window=window)
        assert _ok(got.cpu(), want), (window, ref.max_abs(got.cpu(), want))
    # window 0: the output is exactly the V row of the last token.
    got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                           softmax_scale=0.2, sliding_window=0)
    for bi in range(b):
        n = int(lengths[bi]) - 1
        row = vp[:, int(tables[bi, n // 16]), n % 16]  # [hkv, d]
        assert torch.equal(got[bi].cpu(), row.repeat_interleave(hq // hkv, dim=0))
    rng = np.random.default_rng(17)
    for _ in range(8):
        d = int(rng.choice([64, 128]))
        hkv = int(rng.choice([1, 2, 4]))
        g = int(rng.choice([1, 2, 3, 4, 8, 16]))
        b = int(rng.integers(1, 6))
        pps = int(rng.integers(1, 70))
        window = int(rng.choice([-1, -1, 3, 100]))
        q, kp, vp, tables, lengths = ref.paged_inputs(int(rng.integers(1 << 20)), batch=b, num_heads=hkv * g,
                                                      num_kv_heads=hkv, head_dim=d, page_size=16, pages_per_seq=pps,
                                                      min_len=1, max_len=16 * pps)
        want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=d ** -0.5, page_tables=tables,
                                    sliding_window=None if window < 0 else window)[:, 0]
        got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                               softmax_scale=d ** -0.5, sliding_window=window)
        assert _ok(got.cpu(), want), (b, hkv, g, d, pps, window, ref.max_abs(got.cpu(), want))


# ----------------------------------------------------------------------------- the reference's full decode contract


def _bar(got, want, dtype):
    """The bars of the three dtypes: fp32 1e-5 max-abs; bf16 1e-2 relative L2, float16 an eighth of it."""
    if dtype == torch.float32:
        return got.dtype == dtype and ref.max_abs(got, want) <= 1e-5
    return got.dtype == dtype and ref.rel_l2(got, want) <= (1e-2 if dtype == torch.bfloat16 else 1.25e-3)


def _repage(tables, pool, page_size):
    """The same sequences laid out in pages of `page_size` tokens (a multiple of the 16 of `pool`): the
    new pool's page p of sequence b holds the old logical pages [p * r, (p + 1) * r) of b, the new
    table is a seeded permutation again.  Returns (new pool builder, new tables)."""
    r = page_size // 16
    b, pps = tables.shape
    assert pps % r == 0
    new_pps = pps // r
    perm = torch.from_numpy(np.random.default_rng(11).permutation(b * new_pps).astype(np.int32)).reshape(b, new_pps)

    def build(old):
        hkv, _, _, d = old.shape
        new = torch.empty((hkv, b * new_pps, page_size, d), dtype=old.dtype)
        gathered = old[:, tables.long()]                        # [hkv, b, pps, 16, d]
        new[:, perm.long().reshape(-1)] = gathered.reshape(hkv, b * new_pps, page_size, d)
        return new

    return build, perm


@pytest.mark.parametrize("page_size", [32, 64, 128])
@pytest.mark.parametrize("b,s,h,d", [(1, 1024, 32, 64), (4, 512, 48, 64), (2, 1024, 16, 128), (1, 4096, 8, 128)])
@pytest.mark.parametrize("padding", [0, 111])
@pytest.mark.parametrize("kv_head_factor", [1, 8])
@pytest.mark.parametrize("window", [-1, 127])
def test_paged_decode_page_sizes(page_size, b, s, h, d, padding, kv_head_factor, window):
    """The page sizes the reference admits at its compute block of 128 keys besides 16
    (gpu_paged_attention.py:313-321), on the grid of decoding_test.py:95-163: against the oracle, and -
    with the fixed decomposition - bit for bit against the same tokens in 16-token pages and in a
    contiguous cache (the kernels stream the same 16-token tiles in the same order)."""
    hkv = h // kv_head_factor
    q, kp, vp, tables, _ = ref.paged_inputs(3, batch=b, num_heads=h, num_kv_heads=hkv, head_dim=d, page_size=16,
                                            pages_per_seq=s // 16, min_len=1, max_len=s)
    build, tables2 = _repage(tables, kp, page_size)
    kp2, vp2 = build(kp), build(vp)
    assert torch.equal(ref.reconstruct_kv(tables2, kp2), ref.reconstruct_kv(tables, kp))
    lengths = torch.full((b,), s - padding, dtype=torch.int32)
    scale = d ** -0.5
    want = ref.reference_decode(q, kp2, vp2, lengths, softmax_scale=scale, page_tables=tables2,
                                sliding_window=None if window < 0 else window)[:, 0]
    got = ops.paged_decode(q[:, 0].cuda(), kp2.cuda(), vp2.cuda(), tables2.cuda(), lengths.cuda(),
                           softmax_scale=scale, sliding_window=window)
    assert _ok(got.cpu(), want), ref.rel_l2(got.cpu(), want)
    with _deterministic():
        det = ops.paged_decode(q[:, 0].cuda(), kp2.cuda(), vp2.cuda(), tables2.cuda(), lengths.cuda(),
                               softmax_scale=scale, sliding_window=window)
        det16 = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                                 softmax_scale=scale, sliding_window=window)
    assert torch.equal(det, det16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_paged_decode_page_sizes_ragged_poison_and_dispatch(dtype):
    """Ragged lengths over 64-token pages: tokens past a sequence's length inside its last page, and
    whole pages past it, are never read into the result (NaN poison); the dispatch accepts the pool."""
    b, hq, hkv, d, page, pps = 5, 8, 2, 128, 64, 6
    q, kp, vp, tables, lengths = ref.paged_inputs(19, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=page, pages_per_seq=pps, min_len=1, max_len=page * pps,
                                                  dtype=dtype)
    lengths[0], lengths[1], lengths[2] = 1, page, page + 1
    want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=0.1, page_tables=tables)
    kpo, vpo = kp.clone(), vp.clone()
    for bi in range(b):
        n = int(lengths[bi])
        for j in range(pps):
            lo = max(0, n - j * page)
            if lo < page:
                kpo[:, int(tables[bi, j]), lo:] = float("nan")
                vpo[:, int(tables[bi, j]), lo:] = float("nan")
    tp = (lengths.long() - 1)[:, None].cuda()
    bias = ab.CompositeAttentionBias([ab.CausalAttentionBias(target_positions=tp,
                                                             source_positions=torch.arange(page * pps)[None].cuda())])
    args = dict(query=q.cuda(), key=kpo.cuda(), value=vpo.cuda(), bias=bias)
    impl = flash_attention_implementation("gpu", **args, softmax_scale=0.1, kv_cache_type=PagedKVCache,
                                          page_tables=tables.cuda())
    assert impl is not None and isinstance(impl.fn, HipPagedAttention)
    got = impl.fn(dict(**args, page_tables=tables.cuda()))
    assert torch.isfinite(got.float()).all() and _bar(got.cpu(), want, dtype)
    # the reference's gate: fewer than 16 pages per compute block, the block a multiple of the page
    small = HipPagedAttention.default_config().set(softmax_scale=0.1, gpu_block_size=32).instantiate()
    assert not small.is_supported(dict(**args, page_tables=tables.cuda()), kv_cache_type=PagedKVCache)  # 32 % 64


@pytest.mark.parametrize("g,hkv", [(24, 2), (32, 1), (64, 1), (17, 3)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_decode_more_than_16_query_heads_per_kv_head(g, hkv, dtype):
    """gpu_decoding.py:341 pads its head block to the next power of two, so MQA with 32 or 64 query
    heads runs there; here a kv head's query heads are served in groups of 16."""
    b, d, pps = 3, 128, 24
    hq = g * hkv
    q, kp, vp, tables, lengths = ref.paged_inputs(23, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=1, max_len=16 * pps,
                                                  dtype=dtype)
    want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=0.09, page_tables=tables)[:, 0]
    got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(), softmax_scale=0.09)
    assert _bar(got.cpu(), want, dtype), ref.rel_l2(got.cpu(), want)
    kk, vv = ref.reconstruct_kv(tables, kp).cuda(), ref.reconstruct_kv(tables, vp).cuda()
    got2 = ops.decode(q[:, 0].cuda(), kk, vv, lengths.cuda(), softmax_scale=0.09, sliding_window=-1)
    assert _bar(got2.cpu(), want, dtype)
    # a group's result does not depend on the other groups: heads [16, 2 * 16) alone, as their own call
    if g >= 32 and hkv == 1:
        sub = ops.paged_decode(q[:, 0, 16:32].contiguous().cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                               softmax_scale=0.09, deterministic=True)
        full = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                                softmax_scale=0.09, deterministic=True)
        assert torch.equal(sub, full[:, 16:32])


@pytest.mark.parametrize("d", [8, 40, 72, 80, 96, 120])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_decode_head_dims_between_the_compiled_widths(d, dtype):
    """Any head_dim that is a multiple of 8 up to 128, on the tensors as they are (no padded copies):
    paged pool rows and contiguous cache rows of d elements."""
    b, hq, hkv, pps = 4, 8, 2, 20
    q, kp, vp, tables, lengths = ref.paged_inputs(29, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=1, max_len=16 * pps,
                                                  dtype=dtype)
    scale = d ** -0.5
    for window in (-1, 33):
        want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=scale, page_tables=tables,
                                    sliding_window=None if window < 0 else window)[:, 0]
        got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(),
                               softmax_scale=scale, sliding_window=window)
        assert got.shape == (b, hq, d) and _bar(got.cpu(), want, dtype), (window, ref.rel_l2(got.cpu(), want))
        kk, vv = ref.reconstruct_kv(tables, kp).cuda(), ref.reconstruct_kv(tables, vp).cuda()
        got2 = ops.decode(q[:, 0].cuda(), kk, vv, lengths.cuda(), softmax_scale=scale, sliding_window=window)
        assert _bar(got2.cpu(), want, dtype), window
    # NaNs in the columns of a wider tensor that the call does not cover never reach the result
    wide = torch.full((b, 16 * pps, hkv, d + 8), float("nan"), dtype=dtype)
    wide[..., :d] = ref.reconstruct_kv(tables, kp)
    wide_v = torch.full_like(wide, float("nan"))
    wide_v[..., :d] = ref.reconstruct_kv(tables, vp)
    got3 = ops.decode(q[:, 0].cuda(), wide.cuda()[..., :d], wide_v.cuda()[..., :d], lengths.cuda(),
                      softmax_scale=scale, sliding_window=33)
    assert _bar(got3.cpu(), want, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("bias_shape", ["bh", "1h", "b1"])
@pytest.mark.parametrize("bias_dtype", [torch.float32, torch.bfloat16])
def test_decode_with_an_explicit_bias(dtype, bias_shape, bias_dtype):
    """An explicit bias [B|1, Hq|1, 1, S] beside the causal mask (gpu_decoding.py:327-336,
    gpu_paged_attention.py:346-348), kernel level and through both dispatch classes."""
    b, hq, hkv, d, pps = 3, 8, 2, 128, 18
    s = 16 * pps
    q, kp, vp, tables, lengths = ref.paged_inputs(31, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=1, max_len=s, dtype=dtype)
    lengths[0] = s - 5  # a last tile that straddles the length
    shape = dict(bh=(b, hq, 1, s), **{"1h": (1, hq, 1, s), "b1": (b, 1, 1, s)})[bias_shape]
    dense = (2.0 * ref.normal_tensor(37, shape, torch.float32)).to(bias_dtype)
    want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=0.1, page_tables=tables, dense_bias=dense.float())
    plain = ref.reference_decode(q, kp, vp, lengths, softmax_scale=0.1, page_tables=tables)
    assert ref.rel_l2(plain, want) > 0.1  # the bias matters
    got = ops.paged_decode(q[:, 0].cuda(), kp.cuda(), vp.cuda(), tables.cuda(), lengths.cuda(), softmax_scale=0.1,
                           bias=dense[:, :, 0].cuda())
    assert _bar(got.cpu(), want[:, 0], dtype), ref.rel_l2(got.cpu(), want[:, 0])
    kk, vv = ref.reconstruct_kv(tables, kp).cuda(), ref.reconstruct_kv(tables, vp).cuda()
    got2 = ops.decode(q[:, 0].cuda(), kk, vv, lengths.cuda(), softmax_scale=0.1, bias=dense[:, :, 0].cuda())
    assert _bar(got2.cpu(), want[:, 0], dtype)
    # through the dispatch
    tp = (lengths.long() - 1)[:, None].cuda()
    bias = ab.CompositeAttentionBias([
        ab.CausalAttentionBias(target_positions=tp, source_positions=torch.arange(s)[None].cuda()),
        ab.TensorAttentionBias(dense.cuda()),
    ])
    impl = flash_attention_implementation("gpu", query=q.cuda(), key=kk, value=vv, bias=bias, softmax_scale=0.1,
                                          kv_cache_type=KVCache)
    assert impl is not None and isinstance(impl.fn, HipDecoding)
    assert _bar(impl.fn(dict(query=q.cuda(), key=kk, value=vv, bias=bias)).cpu(), want, dtype)
    pargs = dict(query=q.cuda(), key=kp.cuda(), value=vp.cuda(), bias=bias)
    impl = flash_attention_implementation("gpu", **pargs, softmax_scale=0.1, kv_cache_type=PagedKVCache,
                                          page_tables=tables.cuda())
    assert impl is not None and isinstance(impl.fn, HipPagedAttention)
    assert _bar(impl.fn(dict(**pargs, page_tables=tables.cuda())).cpu(), want, dtype)


def test_decode_with_an_arbitrary_mask_fn():
    """Any mask fn, not only the causal and sliding-window ones (gpu_decoding.py:110,
    gpu_paged_attention.py:108: `mask_fn(kv_len - 1, indices)`): here a strided causal mask."""
    b, hq, hkv, d, pps = 4, 8, 4, 64, 16
    s = 16 * pps
    q, kp, vp, tables, lengths = ref.paged_inputs(41, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=8, max_len=s)
    strided = lambda qp, kp_: (qp >= kp_) & ((qp - kp_) % 3 != 1)
    qpos = (lengths.long() - 1)[:, None]
    keep = strided(qpos, torch.arange(s)[None])                       # [B, S]
    dense = ref.bool_to_bias(keep)[:, None, None, :]                  # [B, 1, 1, S]
    want = ref.reference_decode(q, kp, vp, lengths, softmax_scale=0.2, page_tables=tables, dense_bias=dense)
    tp = qpos.cuda()
    bias = ab.CompositeAttentionBias([ab.MaskFnAttentionBias(strided, target_positions=tp,
                                                             source_positions=torch.arange(s)[None].cuda())])
    kk, vv = ref.reconstruct_kv(tables, kp).cuda(), ref.reconstruct_kv(tables, vp).cuda()
    impl = flash_attention_implementation("gpu", query=q.cuda(), key=kk, value=vv, bias=bias, softmax_scale=0.2,
                                          kv_cache_type=KVCache)
    assert impl is not None and isinstance(impl.fn, HipDecoding)
    got = impl.fn(dict(query=q.cuda(), key=kk, value=vv, bias=bias))
    assert _ok(got.cpu(), want), ref.rel_l2(got.cpu(), want)
    pargs = dict(query=q.cuda(), key=kp.cuda(), value=vp.cuda(), bias=bias)
    impl = flash_attention_implementation("gpu", **pargs, softmax_scale=0.2, kv_cache_type=PagedKVCache,
                                          page_tables=tables.cuda())
    assert impl is not None and isinstance(impl.fn, HipPagedAttention)
    assert _ok(impl.fn(dict(**pargs, page_tables=tables.cuda())).cpu(), want)
    # masking is exact: poison in every key the mask drops changes nothing (fixed decomposition)
    kpo, vpo = ref.reconstruct_kv(tables, kp).clone(), ref.reconstruct_kv(tables, vp).clone()
    for bi in range(b):
        kpo[bi, ~keep[bi]] = 1e4
        vpo[bi, ~keep[bi]] = -1e4
    with _deterministic():
        a = impl_decode = HipDecoding.default_config().set(softmax_scale=0.2).instantiate()
        base = a(dict(query=q.cuda(), key=kk, value=vv, bias=bias))
        poisoned = impl_decode(dict(query=q.cuda(), key=kpo.cuda(), value=vpo.cuda(), bias=bias))
    assert torch.equal(base, poisoned)


@pytest.mark.parametrize("q_dtype,kv_dtype", [(torch.bfloat16, torch.float32), (torch.float32, torch.bfloat16),
                                              (torch.bfloat16, torch.float16)])
def test_decode_kv_dtype_other_than_the_query_dtype(q_dtype, kv_dtype):
    """K/V are cast to the query's dtype (gpu_decoding.py:115,133), so a cache kept in another precision
    is accepted; the result is that of the cast tensors."""
    b, hq, hkv, d, pps = 3, 8, 2, 128, 10
    s = 16 * pps
    q, kp, vp, tables, lengths = ref.paged_inputs(43, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                  page_size=16, pages_per_seq=pps, min_len=1, max_len=s, dtype=kv_dtype)
    q = q.to(q_dtype)
    want = ref.reference_decode(q, kp.to(q_dtype), vp.to(q_dtype), lengths, softmax_scale=0.1, page_tables=tables)
    tp = (lengths.long() - 1)[:, None].cuda()
    bias = ab.CompositeAttentionBias([ab.CausalAttentionBias(target_positions=tp,
                                                             source_positions=torch.arange(s)[None].cuda())])
    pargs = dict(query=q.cuda(), key=kp.cuda(), value=vp.cuda(), bias=bias)
    impl = flash_attention_implementation("gpu", **pargs, softmax_scale=0.1, kv_cache_type=PagedKVCache,
                                          page_tables=tables.cuda())
    assert impl is not None and isinstance(impl.fn, HipPagedAttention)
    got = impl.fn(dict(**pargs, page_tables=tables.cuda()))
    assert _bar(got.cpu(), want, q_dtype)
    kk, vv = ref.reconstruct_kv(tables, kp).cuda(), ref.reconstruct_kv(tables, vp).cuda()
    impl = flash_attention_implementation("gpu", query=q.cuda(), key=kk, value=vv, bias=bias, softmax_scale=0.1,
                                          kv_cache_type=KVCache)
    assert impl is not None and isinstance(impl.fn, HipDecoding)
    assert _bar(impl.fn(dict(query=q.cuda(), key=kk, value=vv, bias=bias)).cpu(), want, q_dtype)
