"""flash_attention/jax_ffi.py, the JAX side of the XLA FFI binding, executed under the stand-ins of
tests/jax_stand_in.py (jax is not installed here): see that module for what this does and does not show."""

import ctypes

import numpy as np
import pytest
import torch

from axlearn_amd import _lib
from axlearn_amd import attention_bias as ab
from axlearn_amd import ops
import jax_stand_in  # tests/jax_stand_in.py (pytest puts the test directory on sys.path)
from oracle import ref_attention as ref

RESIDUAL = "gpu_attention.flash_residuals"   # remat.py:13-58 matches this name


def _size_query(b, t, s, hq, hkv, d, mask_kind, has_seg, flags):
    p = _lib.AxlFlashBwdParams(batch=b, q_len=t, kv_len=s, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, dtype=0,
                               mask_kind=mask_kind, segment_ids=1 if has_seg else None, flags=flags)
    return int(_lib.load().axl_flash_bwd_workspace_bytes(ctypes.byref(p)))


def test_jax_side_imports_and_registers_every_target():
    with jax_stand_in.installed() as (mod, state):
        assert sorted(state.registered) == sorted((t, "ROCM") for t in jax_stand_in.TARGETS)
        for name in ("flash_attention", "HipFlashAttention", "HipDecoding", "HipPagedAttention", "hip_scatter_update_pages"):
            assert hasattr(mod, name)
    import sys

    assert "jax" not in sys.modules and jax_stand_in.JAX_SIDE not in sys.modules and not hasattr(torch.Tensor, "astype")


def test_shim_builds_against_the_stand_in_header_and_checks_its_frame():
    """csrc/ffi_shim.cc compiled against tests/xla_ffi_stand_in (not jaxlib's header, which is absent
    here): the library loads without a GPU, exports a handler per target, and a handler given a frame
    that does not match its binding - operand count, attribute type, attribute name - says so before
    any kernel entry point is reached."""
    shim = jax_stand_in.load_shim()
    for target in jax_stand_in.TARGETS:
        assert hasattr(shim, target)
    x = torch.zeros((2, 4, 8), dtype=torch.bfloat16)
    ok_attrs = dict(softmax_scale=np.float32(1.0), sliding_window=np.int32(-1), flags=np.int32(0))
    with pytest.raises(jax_stand_in.FfiError, match="wrong number of operands") as err:
        jax_stand_in._run_handler("AxlDecode", [x] * 4, [x, x], ok_attrs)
    assert err.value.code == 3
    with pytest.raises(jax_stand_in.FfiError, match="attribute sliding_window has the wrong type"):
        jax_stand_in._run_handler("AxlDecode", [x] * 5, [x, x], dict(ok_attrs, sliding_window=np.float32(-1)))
    renamed = dict(softmax_scale=np.float32(1.0), window=np.int32(-1), flags=np.int32(0))
    with pytest.raises(jax_stand_in.FfiError, match="attribute sliding_window is missing"):
        jax_stand_in._run_handler("AxlDecode", [x] * 5, [x, x], renamed)
    with pytest.raises(TypeError, match="must be np.int32 or np.float32"):
        jax_stand_in._run_handler("AxlDecode", [x] * 5, [x, x], dict(ok_attrs, flags=0))
    # ranks are checked by the handler itself, again before the library is called
    with pytest.raises(jax_stand_in.FfiError, match=r"q must be \[B,Hq,D\]"):
        jax_stand_in._run_handler("AxlDecode", [x] * 5, [x, x], ok_attrs)


@pytest.mark.parametrize("shape,seg,want_flags", [
    ((2, 256, 256, 8, 2, 128), False, 1),            # fits: the dS workspace whole
    ((2, 256, 256, 8, 2, 128), True, 1),
    ((1, 32768, 32768, 64, 8, 128), False, 1 | 2 << 8),  # 69 GB whole: two kv heads at a time under the 18 GB limit
    ((1, 32768, 32768, 32, 1, 128), False, 0),        # 34 GB in one kv head, which cannot be sliced: the recomputing pair
    ((2, 256, 384, 8, 2, 128), False, 1),             # q_len != kv_len: the flag is passed and ignored by the library
])
def test_custom_vjp_pair_sizes_the_workspace_as_the_library_asks(shape, seg, want_flags):
    """The pair given to `defvjp`, with every tensor on the meta device and no kernel run: the forward
    tags out and lse for the remat policy and keeps the residuals of gpu_attention.py:420-424; the
    backward declares a workspace result of exactly axl_flash_bwd_workspace_bytes for the flags it
    chose (whole, in slices of kv heads, or none), and returns no gradient for bias, ids and mask."""
    b, t, s, hq, hkv, d = shape
    with jax_stand_in.installed() as (mod, state):
        state.execute, state.device = False, "meta"
        mk = lambda *dims: torch.empty(dims, dtype=torch.bfloat16, device="meta")
        q, k, v = mk(b, t, hq, d), mk(b, s, hkv, d), mk(b, s, hkv, d)
        ids = torch.empty((b, t), dtype=torch.int64, device="meta") if seg else None
        args = (q, k, v, None, ids, None, None, d ** -0.5, mod.MASK_CAUSAL, 0, 0.0)
        out, pullback = mod.flash_attention.vjp(*args)
        assert state.checkpoint_names == [RESIDUAL, RESIDUAL]
        target, operands, attrs, results = state.calls[0]
        assert target == "AxlFlashFwd" and results == [(b, t, hq, d), (b, hq, t)]
        assert operands[3] == ((b, t) if seg else (0,)) and operands[4:] == [(0,)] * 4
        assert attrs["mask_kind"] == 1 and abs(attrs["softmax_scale"] - d ** -0.5) < 1e-7
        grads = pullback(torch.empty_like(out))
        assert len(grads) == 7 and grads[3:] == (None, None, None, None)
        assert [tuple(g.shape) for g in grads[:3]] == [tuple(x.shape) for x in (q, k, v)]
        target, operands, attrs, results = state.calls[1]
        assert target == "AxlFlashBwd" and attrs["flags"] == want_flags
        want_ws = _size_query(b, t, s, hq, hkv, d, 1, seg, want_flags)
        assert results[3:] == [(0,), (want_ws,)]
        if want_flags >> 8:
            assert want_ws <= mod.BWD_WORKSPACE_LIMIT_BYTES < _size_query(b, t, s, hq, hkv, d, 1, seg, 1)
        # calling the function itself is the forward alone
        n = len(state.calls)
        assert mod.flash_attention(*args).shape == out.shape and len(state.calls) == n + 1


def test_forced_choices_of_the_backward_workspace():
    b, t, hq, hkv, d = 1, 512, 4, 2, 128
    with jax_stand_in.installed() as (mod, state):
        state.execute, state.device = False, "meta"
        mk = lambda h: torch.empty((b, t, h, d), dtype=torch.float16, device="meta")
        args = (mk(hq), mk(hkv), mk(hkv), None, None, None, None, 0.1, mod.MASK_SLIDING_WINDOW, 100, 0.0)
        for forced, flags in ((False, 0), (True, 1)):
            mod.BWD_DS_WORKSPACE = forced
            out, pullback = mod.flash_attention.vjp(*args)
            pullback(torch.empty_like(out))
            assert state.calls[-1][2]["flags"] == flags and state.calls[-1][2]["sliding_window"] == 100
            assert state.calls[-1][3][4] == (_size_query(b, t, t, hq, hkv, d, 2, False, flags),)


def _inputs(b, t, hq, hkv, d, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda h: torch.randn(b, t, h, d, generator=g).to(dtype).cuda()
    return mk(hq), mk(hkv), mk(hkv), mk(hq)


@pytest.mark.gpu
@pytest.mark.parametrize("window,seg", [(None, False), (None, True), (100, True)])
def test_jax_side_flash_attention_runs_the_kernels_like_the_torch_side(window, seg):
    """`HipFlashAttention.__call__` and the custom_vjp pair of the JAX side on the GPU, through the C ABI
    with the buffers the stand-in FFI allocates from the declared result types: bit-identical to
    `ops.flash_fwd` / `ops.flash_bwd` with the torch side's default policy."""
    b, t, hq, hkv, d = 2, 384, 8, 2, 128
    q, k, v, do = _inputs(b, t, hq, hkv, d, torch.bfloat16)
    ids = (torch.arange(t)[None] // torch.tensor([[100], [190]])).int().cuda() + 1 if seg else None
    pos = dict(target_positions=torch.arange(t)[None].cuda(), source_positions=torch.arange(t)[None].cuda())
    mask = ab.CausalAttentionBias(**pos) if window is None else ab.SlidingWindowAttentionBias(
        ab.sliding_window_causal_mask(window), sliding_window_size=window, **pos)
    bias = ab.CompositeAttentionBias([mask] + ([ab.SegmentIdAttentionBias(ids)] if seg else []))
    scale = d ** -0.5
    kw = dict(softmax_scale=scale, mask_kind=ops.MASK_CAUSAL if window is None else ops.MASK_SLIDING_WINDOW,
              sliding_window=window or 0, segment_ids=ids)
    want_out, want_lse = ops.flash_fwd(q, k, v, **kw)
    want = ops.flash_bwd(q, k, v, want_out, want_lse, do, ds_workspace=None, **kw)[:3]
    with jax_stand_in.installed() as (mod, state):
        fa = mod.HipFlashAttention.default_config().set(softmax_scale=scale).instantiate()
        batch = dict(query=q, key=k, value=v, bias=bias)
        assert fa.is_supported(batch, kv_cache_type=None)
        assert torch.equal(fa(batch), want_out)
        assert state.calls[-1][0] == "AxlFlashFwd" and state.calls[-1][2]["mask_kind"] == kw["mask_kind"]
        out, pullback = mod.flash_attention.vjp(q, k, v, None, ids, None, None, scale, kw["mask_kind"], kw["sliding_window"], 0.0)
        assert torch.equal(out, want_out) and state.checkpoint_names == [RESIDUAL, RESIDUAL]
        dq, dk, dv = pullback(do)[:3]
        assert state.calls[-1][2]["flags"] == 1   # the dS workspace fits
        for name, got, exp in (("dq", dq, want[0]), ("dk", dk, want[1]), ("dv", dv, want[2])):
            assert torch.equal(got, exp), name


@pytest.mark.gpu
def test_jax_side_flash_attention_with_bias_and_dropout():
    """An arbitrary mask fn becomes a dense bias once, an explicit bias is added to it, and the dropout
    mask is drawn by the caller: the same operands given to the torch side give the same bits."""
    b, t, hq, hkv, d, rate = 1, 256, 4, 4, 64, 0.25
    q, k, v, do = _inputs(b, t, hq, hkv, d, torch.float16, seed=3)
    pos = dict(target_positions=torch.arange(t)[None].cuda(), source_positions=torch.arange(t)[None].cuda())
    strided = lambda qp, kp: (qp >= kp) & ((qp - kp) % 3 != 1)
    dense = torch.randn(1, hq, t, t, generator=torch.Generator().manual_seed(5)).cuda()
    bias = ab.CompositeAttentionBias([ab.MaskFnAttentionBias(strided, **pos), ab.TensorAttentionBias(dense)])
    with jax_stand_in.installed() as (mod, state):
        fa = mod.HipFlashAttention.default_config().set(softmax_scale=0.125, dropout_rate=rate).instantiate()
        got = fa(dict(query=q, key=k, value=v, bias=bias, prng_key=11))
        import jax  # the stand-in

        drop = jax.random.bernoulli(11, rate, (b, hq, t, t))
        target, operands, attrs, _ = state.calls[-1]
        assert operands[5] == (1, hq, t, t) and operands[6] == (b, hq, t, t) and attrs["mask_kind"] == 0
        assert abs(attrs["dropout_rate"] - rate) < 1e-7
        full = bias.value().float()
        want, lse = ops.flash_fwd(q, k, v, softmax_scale=0.125, mask_kind=ops.MASK_NONE, bias=full,
                                  dropout_mask=drop, dropout_rate=rate)
        assert torch.equal(got, want)
        out, pullback = mod.flash_attention.vjp(q, k, v, full, None, drop, None, 0.125, 0, 0, rate)
        grads = pullback(do)
        exp = ops.flash_bwd(q, k, v, want, lse, do, softmax_scale=0.125, mask_kind=ops.MASK_NONE, bias=full,
                            dropout_mask=drop, dropout_rate=rate)[:3]
        for g, e in zip(grads[:3], exp):
            assert torch.equal(g, e)


@pytest.mark.gpu
def test_jax_side_logit_sink_gets_a_gradient():
    """`logit_sink` is a differentiable argument of the custom_vjp: the forward passes it to the kernel,
    the backward declares the [Hq] result and returns it; same bits as the torch side."""
    b, t, hq, hkv, d = 2, 256, 8, 4, 128
    q, k, v, do = _inputs(b, t, hq, hkv, d, torch.bfloat16, seed=4)
    sink = torch.linspace(-1.0, 2.0, hq).cuda()
    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_CAUSAL, logit_sink=sink)
    want_out, want_lse = ops.flash_fwd(q, k, v, **kw)
    want = ops.flash_bwd(q, k, v, want_out, want_lse, do, ds_workspace=None, **kw)
    assert len(want) == 4
    pos = dict(target_positions=torch.arange(t)[None].cuda(), source_positions=torch.arange(t)[None].cuda())
    bias = ab.CompositeAttentionBias([ab.CausalAttentionBias(**pos)])
    with jax_stand_in.installed() as (mod, state):
        fa = mod.HipFlashAttention.default_config().set(softmax_scale=d ** -0.5).instantiate()
        batch = dict(query=q, key=k, value=v, bias=bias, logit_sink=sink)
        assert fa.is_supported(batch, kv_cache_type=None) and torch.equal(fa(batch), want_out)
        out, pullback = mod.flash_attention.vjp(q, k, v, None, None, None, sink, d ** -0.5, 1, 0, 0.0)
        grads = pullback(do)
        assert state.calls[-1][1][7] == (hq,) and state.calls[-1][3][3] == (hq,)
        for got, exp in zip(grads[:3] + (grads[6],), want):
            assert torch.equal(got, exp)
        assert grads[3:6] == (None, None, None)


@pytest.mark.gpu
def test_jax_side_head_dims_between_the_compiled_widths():
    """head_dim 72 goes to the kernels as it is (16-bit, no bias: `_runs_at_native_head_dim`), with a dense
    bias it is zero-padded to 128 and the output sliced; head_dim 40 with one head (rows closer than a
    compiled width) is padded too.  Each case gives the torch-side class's bits."""
    from axlearn_amd.flash_attention.hip_attention import HipFlashAttention as TorchSide

    for (hq, hkv, d, with_bias) in ((4, 2, 72, False), (4, 2, 72, True), (1, 1, 40, False)):
        b, t = 2, 256
        q, k, v, _ = _inputs(b, t, hq, hkv, d, torch.bfloat16, seed=6)
        pos = dict(target_positions=torch.arange(t)[None].cuda(), source_positions=torch.arange(t)[None].cuda())
        parts = [ab.CausalAttentionBias(**pos)]
        if with_bias:
            parts.append(ab.TensorAttentionBias(torch.randn(1, 1, t, t, generator=torch.Generator().manual_seed(8)).cuda()))
        batch = dict(query=q, key=k, value=v, bias=ab.CompositeAttentionBias(parts))
        torch_side = TorchSide.default_config().set(softmax_scale=0.2).instantiate()
        assert torch_side.is_supported(batch, kv_cache_type=None)
        with torch.no_grad():
            want = torch_side(batch)
        with jax_stand_in.installed() as (mod, state):
            fa = mod.HipFlashAttention.default_config().set(softmax_scale=0.2).instantiate()
            assert fa.is_supported(batch, kv_cache_type=None)
            got = fa(batch)
            native = d == 72 and not with_bias
            assert state.calls[-1][1][0] == (b, t, hq, d if native else (128 if d > 64 else 64))
        assert got.shape == want.shape and torch.equal(got, want)


@pytest.mark.gpu
def test_jax_side_incremental_prefill():
    """`kv_cache_type=KVCache` with a chunk of queries per sequence, each at its own offset into the cache
    (utils_test.py:361-478): rows padded to the 128-row block, offsets passed as the q_pos_offsets
    operand; the torch-side class's bits, for a causal mask and for a window."""
    from axlearn_amd.flash_attention.hip_attention import HipFlashAttention as TorchSide
    from axlearn_amd.kv_cache import KVCache

    b, t, s, hq, hkv, d = 3, 40, 512, 8, 2, 128
    g = torch.Generator().manual_seed(9)
    q = torch.randn(b, t, hq, d, generator=g).to(torch.bfloat16).cuda()
    k = torch.randn(b, s, hkv, d, generator=g).to(torch.bfloat16).cuda()
    v = torch.randn(b, s, hkv, d, generator=g).to(torch.bfloat16).cuda()
    starts = torch.tensor([0, 130, 472])
    pos = dict(target_positions=(starts[:, None] + torch.arange(t)[None]).cuda(), source_positions=torch.arange(s)[None].cuda())
    for window in (None, 64):
        mask = ab.CausalAttentionBias(**pos) if window is None else ab.SlidingWindowAttentionBias(
            ab.sliding_window_causal_mask(window), sliding_window_size=window, **pos)
        batch = dict(query=q, key=k, value=v, bias=ab.CompositeAttentionBias([mask]))
        torch_side = TorchSide.default_config().set(softmax_scale=d ** -0.5).instantiate()
        assert torch_side.is_supported(batch, kv_cache_type=KVCache)
        with torch.no_grad():
            want = torch_side(batch)
        with jax_stand_in.installed() as (mod, state):
            fa = mod.HipFlashAttention.default_config().set(softmax_scale=d ** -0.5).instantiate()
            assert fa.is_supported(batch, kv_cache_type=KVCache)
            got = fa(batch)
            target, operands, attrs, _ = state.calls[-1]
            assert target == "AxlFlashFwd" and operands[0] == (b, 128, hq, d) and operands[7] == (b,)
            assert attrs["mask_kind"] == (1 if window is None else 2) and attrs["sliding_window"] == (window or 0)
        assert got.shape == (b, t, hq, d) and torch.equal(got, want)


@pytest.mark.gpu
def test_jax_side_decode_classes_and_page_insert():
    """`HipDecoding`, `HipPagedAttention` and `hip_scatter_update_pages` of the JAX side against the torch
    side's `ops.decode` / `ops.paged_decode` / `ops.paged_kv_insert` on the same operands: identical bits
    (the deterministic flag is off on both sides, and one call's split is a function of the shapes)."""
    hq, hkv, d, page, pps, b = 8, 2, 128, 16, 8, 3
    qq, kp, vp, tables, lengths = ref.paged_inputs(5, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                    page_size=page, pages_per_seq=pps, min_len=10, max_len=page * pps)
    qq, kp, vp, tables, lengths = (x.cuda() for x in (qq, kp, vp, tables, lengths))
    kv_len = page * pps
    causal = ab.CompositeAttentionBias([ab.CausalAttentionBias(
        target_positions=(lengths.long() - 1)[:, None], source_positions=torch.arange(kv_len)[None].cuda())])
    with jax_stand_in.installed() as (mod, state):
        from axlearn_amd.kv_cache import KVCache, PagedKVCache

        paged = mod.HipPagedAttention.default_config().set(softmax_scale=0.3).instantiate()
        pbatch = dict(query=qq, key=kp, value=vp, bias=causal, page_tables=tables)
        assert paged.is_supported(pbatch, kv_cache_type=PagedKVCache) and not paged.is_supported(pbatch, kv_cache_type=KVCache)
        assert not paged.is_supported(dict(pbatch, key=kp[:, :, :8], value=vp[:, :, :8]), kv_cache_type=PagedKVCache)  # 8-token pages
        got = paged(pbatch)
        want = ops.paged_decode(qq.reshape(b, hq, d), kp, vp, tables, lengths, softmax_scale=0.3)
        assert got.shape == (b, 1, hq, d) and torch.equal(got.reshape(b, hq, d), want)
        # contiguous cache: the same keys gathered
        kk, vv = (ref.reconstruct_kv(tables.cpu(), x.cpu()).contiguous().cuda() for x in (kp, vp))
        dec = mod.HipDecoding.default_config().set(softmax_scale=0.3).instantiate()
        cbatch = dict(query=qq, key=kk, value=vv, bias=causal)
        assert dec.is_supported(cbatch, kv_cache_type=KVCache) and not dec.is_supported(cbatch, kv_cache_type=None)
        assert not dec.is_supported(dict(cbatch, logit_sink=torch.zeros(hq).cuda()), kv_cache_type=KVCache)
        got_c = dec(cbatch)
        want_c = ops.decode(qq.reshape(b, hq, d), kk, vv, lengths, softmax_scale=0.3)
        assert torch.equal(got_c.reshape(b, hq, d), want_c)
        # a mask fn that is neither causal nor a window: evaluated on the host as a row of 0 / NEG_INF
        even = lambda qp, kp_: (kp_ <= qp) & (kp_ % 2 == 0)
        other = ab.CompositeAttentionBias([ab.MaskFnAttentionBias(
            even, target_positions=(lengths.long() - 1)[:, None], source_positions=torch.arange(kv_len)[None].cuda())])
        got_m = dec(dict(query=qq, key=kk, value=vv, bias=other))
        assert state.calls[-1][1][4] == (b, 1, kv_len)
        row = torch.where(even((lengths.long() - 1)[:, None], torch.arange(kv_len)[None].cuda()), 0.0, ab.NEG_INF)
        want_m = ops.decode(qq.reshape(b, hq, d), kk, vv, lengths, softmax_scale=0.3, bias=row[:, None, :].float())
        assert torch.equal(got_m.reshape(b, hq, d), want_m)
        # page insert, in place
        kproj, vproj = torch.randn(2, hkv, b, 1, d, generator=torch.Generator().manual_seed(7)).to(kp.dtype).cuda()
        positions = (lengths - 1).clamp(min=0)
        k2, v2 = kp.clone(), vp.clone()
        ops.paged_kv_insert(k2, v2, kproj[:, :, 0].transpose(0, 1), vproj[:, :, 0].transpose(0, 1), tables, positions)
        k1, v1 = mod.hip_scatter_update_pages(kp, vp, kproj, vproj, tables, positions)
        assert k1.data_ptr() == kp.data_ptr() and torch.equal(k1, k2) and torch.equal(v1, v2)


@pytest.mark.gpu
def test_shim_reports_the_library_errors_as_ffi_errors():
    """A request the library declines comes back as UNIMPLEMENTED with the library's message, a malformed
    one as INVALID_ARGUMENT (`Fail` in the shim): what XLA would raise as an XlaRuntimeError."""
    b, hq, hkv, d = 2, 4, 2, 128
    q = torch.zeros((b, hq, d), dtype=torch.bfloat16, device="cuda")
    pools = torch.zeros((hkv, 8, 8, d), dtype=torch.bfloat16, device="cuda")    # 8-token pages
    tables = torch.zeros((b, 4), dtype=torch.int32, device="cuda")
    lengths = torch.full((b,), 5, dtype=torch.int32, device="cuda")
    none = torch.zeros((0,), device="cuda")
    out, ws = torch.empty_like(q), torch.empty((1 << 20,), dtype=torch.uint8, device="cuda")
    attrs = dict(softmax_scale=np.float32(1.0), sliding_window=np.int32(-1), flags=np.int32(0))
    with pytest.raises(jax_stand_in.FfiError, match="page") as err:
        jax_stand_in._run_handler("AxlPagedDecode", [q, pools, pools, tables, lengths, none], [out, ws], attrs)
    assert err.value.code == 12
    pools16 = torch.zeros((hkv, 8, 16, d), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(jax_stand_in.FfiError, match="workspace") as err:
        jax_stand_in._run_handler("AxlPagedDecode", [q, pools16, pools16, tables, lengths, none], [out, ws[:16]], attrs)
    assert err.value.code == 3
    jax_stand_in._run_handler("AxlPagedDecode", [q, pools16, pools16, tables, lengths, none], [out, ws], attrs)
    torch.cuda.synchronize()
    assert torch.equal(out, torch.zeros_like(out))   # all-zero V rows
