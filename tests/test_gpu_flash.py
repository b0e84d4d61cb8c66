"""GPU parity tests of the flash-attention forward/backward kernels against the CPU oracle.

Tolerances are the ones the task states: fp32 <= 1e-5 max-abs; bf16 (fp32 accumulation) <= 2e-2
max-abs OR <= 1e-2 relative-L2, measured against the oracle's float64 evaluation of the same
bf16-rounded inputs.  Masking is checked bit-exactly through poison tests.
"""

import numpy as np
import pytest
import torch

from axlearn_amd import attention_bias as ab
from axlearn_amd import _lib, ops
from axlearn_amd.flash_attention.hip_attention import HipFlashAttention, flash_attention
from axlearn_amd.flash_attention.utils import flash_attention_implementation
from oracle import brute
from oracle import ref_attention as ref

pytestmark = pytest.mark.gpu

BF16_MAX_ABS, BF16_REL_L2, FP32_MAX_ABS = 2e-2, 1e-2, 1e-5
# float16 carries 3 more mantissa bits than bfloat16: its bar is 8x tighter.
F16_MAX_ABS, F16_REL_L2 = 2.5e-3, 1.25e-3


def _ok_bf16(got, want):
    return ref.max_abs(got, want) <= BF16_MAX_ABS or ref.rel_l2(got, want) <= BF16_REL_L2


def _assert_close(name, got, want, dtype):
    got = got.detach().cpu()
    assert got.dtype == dtype, f"{name}: {got.dtype}"
    if dtype == torch.float32:
        err = ref.max_abs(got, want)
        assert err <= FP32_MAX_ABS, f"{name}: max-abs {err:.3e}"
    elif dtype == torch.float16:
        assert ref.max_abs(got, want) <= F16_MAX_ABS or ref.rel_l2(got, want) <= F16_REL_L2, (
            f"{name}: max-abs {ref.max_abs(got, want):.3e} rel-L2 {ref.rel_l2(got, want):.3e}")
    else:
        assert _ok_bf16(got, want), f"{name}: max-abs {ref.max_abs(got, want):.3e} rel-L2 {ref.rel_l2(got, want):.3e}"
    assert torch.isfinite(got.float()).all(), name


def _inputs(b, t, hq, hkv, d, dtype, s=None):
    s = s or t
    q = ref.normal_tensor(0, (b, t, hq, d), dtype)
    k = ref.normal_tensor(1, (b, s, hkv, d), dtype)
    v = ref.normal_tensor(2, (b, s, hkv, d), dtype)
    do = ref.normal_tensor(3, (b, t, hq, d), dtype)
    return q, k, v, do


def _mask_args(kind, window, seg):
    spec = ref.MaskSpec(causal=kind == "causal", sliding_window=window if kind == "sliding" else None, segment_ids=seg)
    mk = {"none": ops.MASK_NONE, "causal": ops.MASK_CAUSAL, "sliding": ops.MASK_SLIDING_WINDOW}[kind]
    return spec, dict(mask_kind=mk, sliding_window=window or 0, segment_ids=None if seg is None else seg.cuda())


FWD_CASES = [
    # b, t, hq, hkv, d, dtype, mask, window, seg      (shapes follow gpu_attention_test.py:105-130)
    (1, 128, 1, 1, 128, torch.bfloat16, "none", None, False),
    (2, 256, 4, 4, 64, torch.bfloat16, "causal", None, False),
    (1, 384, 8, 2, 128, torch.bfloat16, "causal", None, False),
    (2, 512, 4, 1, 128, torch.bfloat16, "causal", None, True),
    (2, 512, 2, 2, 64, torch.bfloat16, "sliding", 127, False),
    (1, 1024, 4, 2, 128, torch.bfloat16, "sliding", 128, True),
    (1, 1024, 2, 2, 128, torch.bfloat16, "sliding", 129, False),
    (1, 512, 2, 1, 128, torch.bfloat16, "sliding", 0, False),
    (1, 256, 2, 2, 128, torch.bfloat16, "none", None, True),
    # float16, as the reference's tests run (gpu_attention_test.py:122)
    (2, 256, 4, 4, 64, torch.float16, "causal", None, False),
    (1, 384, 8, 2, 128, torch.float16, "causal", None, True),
    (1, 1024, 4, 2, 128, torch.float16, "sliding", 128, False),
    (1, 256, 2, 1, 128, torch.float16, "none", None, False),
    (2, 512, 4, 4, 64, torch.float32, "causal", None, False),  # BASELINE config 1
    (1, 256, 4, 2, 128, torch.float32, "sliding", 100, True),
    (1, 256, 2, 2, 64, torch.float32, "none", None, False),
]


@pytest.mark.parametrize("b,t,hq,hkv,d,dtype,mask,window,seg", FWD_CASES)
def test_forward_matches_oracle(b, t, hq, hkv, d, dtype, mask, window, seg):
    q, k, v, _ = _inputs(b, t, hq, hkv, d, dtype)
    segs = ref.packed_segment_ids(4, b, t, max_docs=5) if seg else None
    spec, kw = _mask_args(mask, window, segs)
    scale = d ** -0.5
    want, want_lse = ref.reference_mha(q, k, v, spec, softmax_scale=scale, return_lse=True)
    out, lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), softmax_scale=scale, **kw)
    _assert_close("out", out, want, dtype)
    assert ref.max_abs(lse.cpu(), want_lse) < (1e-5 if dtype == torch.float32 else 1e-3) * max(1.0, float(want_lse.abs().max()))
    if dtype == torch.bfloat16:
        # The dtype-faithful restatement (reference rounding points) is as close as the float64 one.
        faithful = ref.reference_mha(q, k, v, spec, softmax_scale=scale, mode="faithful")
        assert _ok_bf16(out.cpu(), faithful)


def test_forward_kv_longer_than_q_and_scale_one():
    q, k, v, _ = _inputs(1, 128, 2, 1, 128, torch.bfloat16, s=384)
    want = ref.reference_mha(q * 0.1, k, v, None, softmax_scale=1.0)
    out, _ = ops.flash_fwd((q * 0.1).cuda(), k.cuda(), v.cuda(), softmax_scale=1.0)
    _assert_close("out", out, ref.reference_mha((q * 0.1), k, v, None, softmax_scale=1.0), torch.bfloat16)
    del want


BWD_CASES = [
    (1, 128, 1, 1, 128, "none", None, False),
    (2, 256, 4, 4, 64, "causal", None, False),
    (1, 384, 8, 2, 128, "causal", None, False),
    (2, 512, 4, 1, 128, "causal", None, True),
    (1, 1024, 4, 2, 128, "sliding", 300, True),
    (2, 512, 2, 2, 64, "sliding", 127, False),
    # long enough for every kind of loop run in the backward kernels: masked tiles at the window edge,
    # mask-free interior tiles, masked diagonal tiles; odd and even numbers of 64-key tiles
    (1, 2048, 2, 1, 128, "sliding", 600, False),
    (1, 2048, 2, 2, 128, "sliding", 40, False),
    (1, 1920, 2, 1, 64, "sliding", 777, False),
    (1, 1536, 4, 2, 128, "none", None, False),
    (1, 1664, 4, 2, 64, "causal", None, False),
    (1, 1152, 2, 1, 128, "sliding", 1000, True),
]


@pytest.mark.parametrize("b,t,hq,hkv,d,mask,window,seg", BWD_CASES)
def test_backward_matches_oracle(b, t, hq, hkv, d, mask, window, seg):
    dtype = torch.bfloat16
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype)
    segs = ref.packed_segment_ids(4, b, t, max_docs=5) if seg else None
    spec, kw = _mask_args(mask, window, segs)
    scale = d ** -0.5
    wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=scale)
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    out, lse = ops.flash_fwd(qc, kc, vc, softmax_scale=scale, **kw)
    _assert_close("out", out, ref.reference_mha(q, k, v, spec, softmax_scale=scale), dtype)
    dq, dk, dv = ops.flash_bwd(qc, kc, vc, out, lse, doc, softmax_scale=scale, **kw)
    if hq * t >= 16384:
        # dk / dv of the two large cases sum a thousand rows of several heads into elements of magnitude
        # 3 to 10, whose fp32 spacing alone is up to 1e-6: the bar scales with the largest element there.
        for name, got, want in (("dq", dq, wq), ("dk", dk, wk), ("dv", dv, wv)):
            err, top = ref.max_abs(got.cpu(), want), float(want.abs().max())
            assert err <= FP32_MAX_ABS * max(1.0, top), f"{name}: max-abs {err:.3e}, largest element {top:.2f}"
    else:
        _assert_close("dq", dq, wq, dtype)
        _assert_close("dk", dk, wk, dtype)
        _assert_close("dv", dv, wv, dtype)


@pytest.mark.parametrize("b,t,hq,hkv,d,mask,window,seg", [
    (2, 256, 4, 4, 64, "causal", None, False),
    (1, 384, 8, 2, 128, "causal", None, True),
    (1, 1024, 4, 2, 128, "sliding", 300, True),
    (1, 1536, 4, 2, 128, "none", None, False),
    (1, 1920, 2, 1, 64, "sliding", 777, False),
])
def test_float16_backward_matches_oracle(b, t, hq, hkv, d, mask, window, seg):
    """float16 forward + backward (gpu_attention_test.py:197 runs float16 and float32), all phases in
    one call and phase by phase (the separate delta pre-pass)."""
    dtype = torch.float16
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype)
    segs = ref.packed_segment_ids(4, b, t, max_docs=5) if seg else None
    spec, kw = _mask_args(mask, window, segs)
    scale = d ** -0.5
    wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=scale)
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    out, lse = ops.flash_fwd(qc, kc, vc, softmax_scale=scale, **kw)
    _assert_close("out", out, ref.reference_mha(q, k, v, spec, softmax_scale=scale), dtype)
    dq, dk, dv = ops.flash_bwd(qc, kc, vc, out, lse, doc, softmax_scale=scale, **kw)
    if hq * t >= 16384:
        # dk / dv of the two large cases sum a thousand rows of several heads into elements of magnitude
        # 3 to 10, whose fp32 spacing alone is up to 1e-6: the bar scales with the largest element there.
        for name, got, want in (("dq", dq, wq), ("dk", dk, wk), ("dv", dv, wv)):
            err, top = ref.max_abs(got.cpu(), want), float(want.abs().max())
            assert err <= FP32_MAX_ABS * max(1.0, top), f"{name}: max-abs {err:.3e}, largest element {top:.2f}"
    else:
        _assert_close("dq", dq, wq, dtype)
        _assert_close("dk", dk, wk, dtype)
        _assert_close("dv", dv, wv, dtype)
    bufs = (torch.zeros_like(dq), torch.zeros_like(dk), torch.zeros_like(dv),
            ops.flash_bwd_buffers(qc, kc, vc, mask_kind=kw["mask_kind"], segment_ids=kw.get("segment_ids"))[3])
    for phase in (1, 2, 4):  # delta, dK/dV, dQ
        ops.flash_bwd(qc, kc, vc, out, lse, doc, softmax_scale=scale, phases=phase, buffers=bufs, **kw)
    _assert_close("dq by phases", bufs[0], wq, dtype)
    _assert_close("dk by phases", bufs[1], wk, dtype)
    _assert_close("dv by phases", bufs[2], wv, dtype)


@pytest.mark.parametrize("b,t,s,hq,hkv,d,mask,window,seg", [
    (2, 512, 512, 4, 4, 64, "causal", None, False),      # BASELINE config 1, with its backward
    (1, 256, 256, 4, 2, 128, "sliding", 100, True),
    (1, 384, 384, 8, 2, 128, "causal", None, True),
    (2, 256, 256, 2, 2, 64, "none", None, False),
    (1, 128, 384, 2, 1, 128, "none", None, False),
    (1, 640, 640, 2, 1, 64, "sliding", 33, False),
    (1, 256, 512, 4, 2, 64, "causal", None, False),
    # enough 256-row blocks for every CU: the forward runs its workgroups of eight wavefronts
    (2, 1024, 1024, 32, 8, 128, "causal", None, False),
    (4, 512, 512, 32, 32, 64, "sliding", 100, True),
])
def test_float32_backward_matches_oracle(b, t, s, hq, hkv, d, mask, window, seg):
    """float32 forward + backward (gpu_attention_test.py:197 runs float16 and float32; the reference
    shrinks its backward blocks for float32, gpu_attention.py:645-646), against the float64 oracle at
    the fp32 bar, all phases in one call and phase by phase (bit-identical: same kernels)."""
    dtype = torch.float32
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype, s=s)
    segs = ref.packed_segment_ids(4, b, t, max_docs=5) if seg else None
    spec, kw = _mask_args(mask, window, segs)
    scale = d ** -0.5
    wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=scale)
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    out, lse = ops.flash_fwd(qc, kc, vc, softmax_scale=scale, **kw)
    _assert_close("out", out, ref.reference_mha(q, k, v, spec, softmax_scale=scale), dtype)
    dq, dk, dv = ops.flash_bwd(qc, kc, vc, out, lse, doc, softmax_scale=scale, **kw)
    if hq * t >= 16384:
        # dk / dv of the two large cases sum a thousand rows of several heads into elements of magnitude
        # 3 to 10, whose fp32 spacing alone is up to 1e-6: the bar scales with the largest element there.
        for name, got, want in (("dq", dq, wq), ("dk", dk, wk), ("dv", dv, wv)):
            err, top = ref.max_abs(got.cpu(), want), float(want.abs().max())
            assert err <= FP32_MAX_ABS * max(1.0, top), f"{name}: max-abs {err:.3e}, largest element {top:.2f}"
    else:
        _assert_close("dq", dq, wq, dtype)
        _assert_close("dk", dk, wk, dtype)
        _assert_close("dv", dv, wv, dtype)
    bufs = (torch.zeros_like(dq), torch.zeros_like(dk), torch.zeros_like(dv),
            ops.flash_bwd_buffers(qc, kc, vc, mask_kind=kw["mask_kind"], segment_ids=kw.get("segment_ids"))[3])
    for phase in (1, 2, 4):  # delta, dK/dV, dQ
        ops.flash_bwd(qc, kc, vc, out, lse, doc, softmax_scale=scale, phases=phase, buffers=bufs, **kw)
    assert torch.equal(bufs[0], dq) and torch.equal(bufs[1], dk) and torch.equal(bufs[2], dv)


def test_float32_kernels_on_the_fp32_matrix_instruction_agree():
    """The library keeps its first fp32 kernels (v_mfma_f32_32x32x2_f32) behind AXL_F32_MFMA=1, read once per
    process: a child process runs them on the inputs this process gives the default kernels (fp32 products
    from split bf16 operands); forward, lse and gradients agree to the fp32 bar (scaled by the largest
    element for the gradients, which sum hundreds of rows)."""
    import os
    import subprocess
    import sys
    import tempfile

    b, t, hq, hkv, d = 1, 512, 8, 2, 128
    q, k, v, do = (x.cuda() for x in _inputs(b, t, hq, hkv, d, torch.float32))
    segs = ref.packed_segment_ids(4, b, t, max_docs=3).cuda()
    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_SLIDING_WINDOW, sliding_window=300, segment_ids=segs)
    out, lse = ops.flash_fwd(q, k, v, **kw)
    mine = [out, lse] + list(ops.flash_bwd(q, k, v, out, lse, do, **kw)[:3])
    child = (
        "import sys, torch\n"
        "from axlearn_amd import ops\n"
        "x = torch.load(sys.argv[1], weights_only=True)\n"
        "kw = dict(softmax_scale=x['scale'], mask_kind=ops.MASK_SLIDING_WINDOW, sliding_window=300, segment_ids=x['segs'].cuda())\n"
        "q, k, v, do = (x[n].cuda() for n in ('q', 'k', 'v', 'do'))\n"
        "out, lse = ops.flash_fwd(q, k, v, **kw)\n"
        "res = [out, lse] + list(ops.flash_bwd(q, k, v, out, lse, do, **kw)[:3])\n"
        "torch.save([r.cpu() for r in res], sys.argv[2])\n"
    )
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with tempfile.TemporaryDirectory() as tmp:
        src, dst = os.path.join(tmp, "in.pt"), os.path.join(tmp, "out.pt")
        torch.save(dict(q=q.cpu(), k=k.cpu(), v=v.cpu(), do=do.cpu(), segs=segs.cpu(), scale=d ** -0.5), src)
        env = dict(os.environ, AXL_F32_MFMA="1", PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
        subprocess.run([sys.executable, "-c", child, src, dst], check=True, env=env, timeout=110, cwd=root)
        theirs = torch.load(dst, weights_only=True)
    for name, a, c in zip(("out", "lse", "dq", "dk", "dv"), mine, theirs):
        err, top = ref.max_abs(a.cpu(), c.double()), float(c.abs().max())
        assert err <= 2 * FP32_MAX_ABS * max(1.0, top), f"{name}: the two kernel families differ by {err:.3e} (largest element {top:.2f})"
        assert not torch.equal(a.cpu(), c) or name == "lse", f"{name}: identical bits - the child did not run the other kernels"


@pytest.mark.parametrize("mask,window", [("causal", None), ("sliding", 333)])
@pytest.mark.parametrize("d", [64, 128])
def test_backward_with_more_keys_than_queries(mask, window, d):
    """A chunk of T queries at positions q_off .. q_off+T-1 over S > T keys (gradients of an incremental
    prefill): dq, dk, dv against the oracle with explicit query positions."""
    b, t, s_len, hq, hkv, q_off = 1, 256, 1024, 4, 2, 640
    dtype = torch.bfloat16
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype, s=s_len)
    spec = ref.MaskSpec(causal=mask == "causal", sliding_window=window,
                        target_positions=torch.arange(q_off, q_off + t)[None], source_positions=torch.arange(s_len)[None])
    mk = ops.MASK_CAUSAL if mask == "causal" else ops.MASK_SLIDING_WINDOW
    kw = dict(mask_kind=mk, sliding_window=window or 0, q_pos_offset=q_off, softmax_scale=d ** -0.5)
    wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=d ** -0.5)
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    out, lse = ops.flash_fwd(qc, kc, vc, **kw)
    _assert_close("out", out, ref.reference_mha(q, k, v, spec, softmax_scale=d ** -0.5), dtype)
    dq, dk, dv = ops.flash_bwd(qc, kc, vc, out, lse, doc, **kw)
    _assert_close("dq", dq, wq, dtype)
    _assert_close("dk", dk, wk, dtype)
    _assert_close("dv", dv, wv, dtype)


@pytest.mark.parametrize("seed", list(range(12)))
def test_random_shapes_forward_and_backward(seed):
    """Seeded sweep over sequence lengths (queries and keys), head layouts, head dims, mask kinds,
    window sizes, query offsets and packings: out, dq, dk, dv against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    d = int(rng.choice([64, 128]))
    hkv = int(rng.choice([1, 2]))
    hq = hkv * int(rng.choice([1, 2, 4]))
    t = 128 * int(rng.integers(1, 8))
    kind = str(rng.choice(["none", "causal", "sliding"]))
    packed = bool(rng.integers(0, 2))
    extra = 0 if packed else 128 * int(rng.integers(0, 4))     # segment ids need S == T
    s_len = t + extra
    q_off = 0 if kind == "none" else extra                     # the chunk ends where the keys end
    window = int(rng.integers(0, s_len)) if kind == "sliding" else None
    dtype = torch.bfloat16
    q, k, v, do = _inputs(1, t, hq, hkv, d, dtype, s=s_len)
    segs = ref.packed_segment_ids(seed, 1, t, max_docs=4) if packed else None
    spec = ref.MaskSpec(causal=kind == "causal", sliding_window=window, segment_ids=segs,
                        target_positions=torch.arange(q_off, q_off + t)[None],
                        source_positions=torch.arange(s_len)[None])
    mk = {"none": ops.MASK_NONE, "causal": ops.MASK_CAUSAL, "sliding": ops.MASK_SLIDING_WINDOW}[kind]
    kw = dict(mask_kind=mk, sliding_window=window or 0, q_pos_offset=q_off, softmax_scale=d ** -0.5,
              segment_ids=None if segs is None else segs.cuda())
    case = f"d={d} hq={hq} hkv={hkv} t={t} s={s_len} {kind} window={window} packed={packed} q_off={q_off}"
    want = ref.reference_mha(q, k, v, spec, softmax_scale=d ** -0.5)
    wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=d ** -0.5)
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    out, lse = ops.flash_fwd(qc, kc, vc, **kw)
    _assert_close("out " + case, out, want, dtype)
    dq, dk, dv = ops.flash_bwd(qc, kc, vc, out, lse, doc, **kw)
    _assert_close("dq " + case, dq, wq, dtype)
    _assert_close("dk " + case, dk, wk, dtype)
    _assert_close("dv " + case, dv, wv, dtype)


@pytest.mark.parametrize("seed", range(8))
def test_random_shapes_with_pairs_spread_over_xcds(seed):
    """Shapes whose (batch x kv head) pairs are a multiple of 8, which the kernels work through in
    per-XCD groups (including a last group smaller than the others): out, dq, dk, dv against the
    oracle, bf16 and fp16, every mask kind, with and without packing."""
    rng = np.random.default_rng(5000 + seed)
    d = int(rng.choice([64, 128]))
    b, hkv = [(1, 8), (2, 4), (3, 8), (8, 1), (2, 8), (5, 8)][int(rng.integers(0, 6))]
    hq = hkv * int(rng.choice([1, 2, 4]))
    t = 128 * int(rng.integers(1, 10))
    kind = str(rng.choice(["none", "causal", "sliding"]))
    packed = bool(rng.integers(0, 2))
    dtype = [torch.bfloat16, torch.float16][int(rng.integers(0, 2))]
    window = int(rng.integers(0, t)) if kind == "sliding" else None
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype, s=t)
    segs = ref.packed_segment_ids(seed, b, t, max_docs=4) if packed else None
    spec = ref.MaskSpec(causal=kind == "causal", sliding_window=window, segment_ids=segs,
                        target_positions=torch.arange(t)[None], source_positions=torch.arange(t)[None])
    mk = {"none": ops.MASK_NONE, "causal": ops.MASK_CAUSAL, "sliding": ops.MASK_SLIDING_WINDOW}[kind]
    kw = dict(mask_kind=mk, sliding_window=window or 0, q_pos_offset=0, softmax_scale=d ** -0.5,
              segment_ids=None if segs is None else segs.cuda())
    case = f"b={b} d={d} hq={hq} hkv={hkv} t={t} {kind} window={window} packed={packed} {dtype}"
    want = ref.reference_mha(q, k, v, spec, softmax_scale=d ** -0.5)
    wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=d ** -0.5)
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    out, lse = ops.flash_fwd(qc, kc, vc, **kw)
    _assert_close("out " + case, out, want, dtype)
    dq, dk, dv = ops.flash_bwd(qc, kc, vc, out, lse, doc, **kw)
    _assert_close("dq " + case, dq, wq, dtype)
    _assert_close("dk " + case, dk, wk, dtype)
    _assert_close("dv " + case, dv, wv, dtype)


@pytest.mark.parametrize("mask,window", [("none", None), ("causal", None), ("sliding", 200)])
def test_arbitrary_segment_ids_forward_and_backward(mask, window):
    """Segment ids are compared for equality only (attention_bias.py:876-882): ids need not be sorted,
    contiguous or non-zero.  Random ids in {0..3} changing every 1..40 positions mask most tiles
    partially and some wholly, which is what the kernels' segment pruning has to survive."""
    b, t, hq, hkv, d = 2, 768, 4, 2, 128
    rng = np.random.default_rng(11)
    seg = np.zeros((b, t), dtype=np.int32)
    for bi in range(b):
        pos = 0
        while pos < t:
            n = int(rng.integers(1, 41))
            seg[bi, pos:pos + n] = int(rng.integers(0, 4))
            pos += n
    seg[1, 256:512] = 7                      # one id that fills whole tiles
    segs = torch.from_numpy(seg)
    q, k, v, do = _inputs(b, t, hq, hkv, d, torch.bfloat16)
    spec, kw = _mask_args(mask, window, segs)
    scale = d ** -0.5
    want = ref.reference_mha(q, k, v, spec, softmax_scale=scale)
    wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=scale)
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    out, lse = ops.flash_fwd(qc, kc, vc, softmax_scale=scale, **kw)
    _assert_close("out", out, want, torch.bfloat16)
    dq, dk, dv = ops.flash_bwd(qc, kc, vc, out, lse, doc, softmax_scale=scale, **kw)
    _assert_close("dq", dq, wq, torch.bfloat16)
    _assert_close("dk", dk, wk, torch.bfloat16)
    _assert_close("dv", dv, wv, torch.bfloat16)


def test_query_offset_chunk_against_full_prefill():
    """Incremental prefill: a chunk of queries at positions q_off .. q_off+T-1 over S > T keys equals
    the same rows of a full causal / sliding-window prefill, bit for bit (same tiles, same order)."""
    b, s_len, hq, hkv, d, t, q_off = 1, 512, 4, 2, 128, 128, 384
    q, k, v, _ = _inputs(b, s_len, hq, hkv, d, torch.bfloat16)
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    for kw in (dict(mask_kind=ops.MASK_CAUSAL), dict(mask_kind=ops.MASK_SLIDING_WINDOW, sliding_window=150)):
        full, full_lse = ops.flash_fwd(qc, kc, vc, softmax_scale=d ** -0.5, **kw)
        part, part_lse = ops.flash_fwd(qc[:, q_off:q_off + t].contiguous(), kc, vc, softmax_scale=d ** -0.5,
                                       q_pos_offset=q_off, **kw)
        assert torch.equal(part, full[:, q_off:q_off + t])
        assert torch.equal(part_lse, full_lse[:, :, q_off:q_off + t])


def test_against_c_brute_force_tiny():
    """Independent loop-level checker (oracle/brute_force.c) incl. GQA, window and segments."""
    b, t, hq, hkv, d = 1, 128, 2, 1, 64
    q, k, v, do = _inputs(b, t, hq, hkv, d, torch.bfloat16)
    segs = ref.packed_segment_ids(9, b, t, max_docs=3)
    scale = 0.2
    bo, bl = brute.attention_fwd(q.float().numpy(), k.float().numpy(), v.float().numpy(), scale=scale,
                                 mask_kind=brute.MASK_SLIDING, window=40, segment_ids=segs.numpy())
    bq, bk, bv = brute.attention_bwd(q.float().numpy(), k.float().numpy(), v.float().numpy(), do.float().numpy(),
                                     scale=scale, mask_kind=brute.MASK_SLIDING, window=40, segment_ids=segs.numpy())
    kw = dict(softmax_scale=scale, mask_kind=ops.MASK_SLIDING_WINDOW, sliding_window=40, segment_ids=segs.cuda())
    out, lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), **kw)
    dq, dk, dv = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), **kw)
    for name, got, want in (("out", out, bo), ("dq", dq, bq), ("dk", dk, bk), ("dv", dv, bv)):
        _assert_close(name, got, torch.from_numpy(want), torch.bfloat16)
    assert np.abs(lse.cpu().numpy() - bl).max() < 1e-3


def test_masking_is_exact_poison():
    """Masked keys must not influence anything: huge garbage planted in K/V rows that every query
    of another segment (or outside the window) ignores leaves those queries' outputs bit-identical.
    The garbage is finite on purpose: the reference masks additively (logit + -1e15) and multiplies
    the resulting exact-zero probability with V, so a NaN in a masked row of a partially visible
    tile would propagate through 0 * NaN in the reference's kernels and XLA path alike."""
    poison = 1e30
    b, t, h, d = 1, 512, 2, 128
    q, k, v, do = _inputs(b, t, h, h, d, torch.bfloat16)
    seg = torch.ones((b, t), dtype=torch.int32)
    seg[:, 200:330] = 2
    seg[:, 330:] = 3
    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_CAUSAL, segment_ids=seg.cuda())
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    out0, lse0 = ops.flash_fwd(qc, kc, vc, **kw)
    dq0, dk0, dv0 = ops.flash_bwd(qc, kc, vc, out0, lse0, doc, **kw)
    kp, vp = kc.clone(), vc.clone()
    kp[:, 200:330] = poison
    vp[:, 200:330] = poison
    out1, lse1 = ops.flash_fwd(qc, kp, vp, **kw)
    keep = (seg[0] != 2).cuda()
    assert torch.equal(out0[:, keep], out1[:, keep]) and torch.equal(lse0[:, :, keep], lse1[:, :, keep])
    assert torch.isfinite(out1[:, keep].float()).all()
    # Backward: poison the OTHER segments' queries' upstream gradient instead (dO rows of segment 2):
    # dK/dV of segments 1 and 3 must not change, dQ rows of segments 1 and 3 neither.
    dop = doc.clone()
    dop[:, 200:330] = 7.0
    dq1, dk1, dv1 = ops.flash_bwd(qc, kc, vc, out0, lse0, dop, **kw)
    assert torch.equal(dq0[:, keep], dq1[:, keep])
    assert torch.equal(dk0[:, keep], dk1[:, keep]) and torch.equal(dv0[:, keep], dv1[:, keep])
    # Sliding window: keys further than w to the left are never read by late queries.
    w = 100
    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_SLIDING_WINDOW, sliding_window=w)
    out0, _ = ops.flash_fwd(qc, kc, vc, **kw)
    kp, vp = kc.clone(), vc.clone()
    kp[:, :128] = poison
    vp[:, :128] = poison
    out1, _ = ops.flash_fwd(qc, kp, vp, **kw)
    assert torch.equal(out0[:, 127 + w + 1:], out1[:, 127 + w + 1:])
    # Causal: the future never leaks.
    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_CAUSAL)
    out0, _ = ops.flash_fwd(qc, kc, vc, **kw)
    kp, vp = kc.clone(), vc.clone()
    kp[:, 300:] = poison
    vp[:, 300:] = poison
    out1, _ = ops.flash_fwd(qc, kp, vp, **kw)
    assert torch.equal(out0[:, :300], out1[:, :300])


def test_closed_forms_and_determinism():
    b, t, h, d = 1, 256, 2, 128
    q, k, v, do = _inputs(b, t, h, h, d, torch.bfloat16)
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_CAUSAL)
    out, lse = ops.flash_fwd(qc, kc, vc, **kw)
    assert torch.equal(out[:, 0], vc[:, 0])  # causal row 0 == V[0]
    out_w0, _ = ops.flash_fwd(qc, kc, vc, softmax_scale=1.0, mask_kind=ops.MASK_SLIDING_WINDOW, sliding_window=0)
    assert torch.equal(out_w0, vc)  # window 0 == self only
    const = torch.ones_like(vc) * 0.5
    out_c, _ = ops.flash_fwd(qc, kc, const, **kw)
    assert torch.equal(out_c, const)  # uniform V
    # Bitwise run-to-run determinism (no atomics anywhere), forward and backward.
    out2, lse2 = ops.flash_fwd(qc, kc, vc, **kw)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)
    g1 = ops.flash_bwd(qc, kc, vc, out, lse, do.cuda(), **kw)
    g2 = ops.flash_bwd(qc, kc, vc, out, lse, do.cuda(), **kw)
    for a, c in zip(g1, g2):
        assert torch.equal(a, c)


@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 128), (torch.float16, 64), (torch.bfloat16, 72)])
@pytest.mark.parametrize("mask,seg", [("causal", False), ("causal", True), ("window", False), ("window", True), ("none", False)])
def test_results_do_not_depend_on_what_ran_before(dtype, d, mask, seg):
    """The same call three times, with other kernels and freshly dirtied workspaces in between: identical
    bits, for the recomputing backward, the dS-workspace backward whole and in slices of kv heads, and the
    forward.  A register read too early behind an assembly MFMA chain shows up exactly here: as values
    that change from run to run."""
    b, t, hq, hkv = 2, 1024, 8, 2
    q, k, v, do = (x.cuda() for x in _inputs(b, t, hq, hkv, d, dtype))
    segs = ref.packed_segment_ids(11, b, t, max_docs=4).cuda() if seg else None
    kw = dict(softmax_scale=d ** -0.5, segment_ids=segs,
              mask_kind={"causal": ops.MASK_CAUSAL, "window": ops.MASK_SLIDING_WINDOW, "none": ops.MASK_NONE}[mask],
              sliding_window=300 if mask == "window" else 0)
    runs = []
    for i in range(3):
        dirt = torch.full((48 << 20,), float(i) - 1.5, device="cuda")   # what the next allocations will find
        del dirt
        out, lse = ops.flash_fwd(q, k, v, **kw)
        grads = [out, lse]
        for ds, heads in ((False, 0), (True, 0), (True, 1)):
            grads += list(ops.flash_bwd(q, k, v, out, lse, do, ds_workspace=ds, ds_slice_kv_heads=heads, **kw)[:3])
        torch.cuda.synchronize()
        runs.append([x.clone() for x in grads])
        _ = torch.randn(1 << 20, device="cuda").sort()   # something else on the GPU in between
    for other in runs[1:]:
        for i, (a, c) in enumerate(zip(runs[0], other)):
            assert torch.equal(a, c), f"result {i} differs between runs"
    # and the three backward forms agree with each other on dk / dv bit for bit where they share the kernel
    dq_r, dk_r, dv_r, dq_w, dk_w, dv_w, dq_s, dk_s, dv_s = runs[0][2:]
    assert torch.equal(dk_w, dk_s) and torch.equal(dv_w, dv_s) and torch.equal(dq_w, dq_s)


def test_strided_inputs():
    """q/k/v sliced out of one fused [B,T,H+2Hkv,D] projection (non-contiguous heads stride)."""
    b, t, hq, hkv, d = 1, 256, 4, 2, 128
    fused = ref.normal_tensor(5, (b, t, hq + 2 * hkv, d), torch.bfloat16).cuda()
    q, k, v = fused[:, :, :hq], fused[:, :, hq:hq + hkv], fused[:, :, hq + hkv:]
    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_CAUSAL)
    out, lse = ops.flash_fwd(q, k, v, **kw)
    out_c, lse_c = ops.flash_fwd(q.contiguous(), k.contiguous(), v.contiguous(), **kw)
    assert torch.equal(out, out_c) and torch.equal(lse, lse_c)
    do = torch.randn_like(out)
    g = ops.flash_bwd(q, k, v, out, lse, do, **kw)
    gc = ops.flash_bwd(q.contiguous(), k.contiguous(), v.contiguous(), out, lse, do, **kw)
    for a, c in zip(g, gc):
        assert torch.equal(a, c)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_dispatch_and_autograd_end_to_end(dtype):
    b, t, hq, hkv, d = 2, 256, 4, 2, 128
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype)
    segs = ref.packed_segment_ids(4, b, t, max_docs=3)
    pos = dict(target_positions=torch.arange(t)[None], source_positions=torch.arange(t)[None])
    bias = ab.CompositeAttentionBias([
        ab.SlidingWindowAttentionBias(ab.sliding_window_causal_mask(64), sliding_window_size=64, **pos),
        ab.SegmentIdAttentionBias(segs.cuda()),
    ])
    qd, kd, vd = (x.cuda().requires_grad_(True) for x in (q, k, v))
    scale = d ** -0.5
    impl = flash_attention_implementation("gpu", query=qd, key=kd, value=vd, bias=bias, softmax_scale=scale)
    assert impl is not None and isinstance(impl.fn, HipFlashAttention)
    out = impl.fn(dict(query=qd, key=kd, value=vd, bias=bias))
    # Same loss as the reference's tests: mean of the output (gpu_attention_test.py:59-92); with
    # float16 it is scaled up, as float16 training does, so that d_out = 1/numel is a normal number.
    loss_scale = 2.0 ** 14 if dtype == torch.float16 else 1.0
    (out.float().mean() * loss_scale).backward()
    spec = ref.MaskSpec(sliding_window=64, segment_ids=segs)
    want = ref.reference_mha(q, k, v, spec, softmax_scale=scale)
    ones = torch.full_like(want, loss_scale / want.numel())
    wq, wk, wv = ref.reference_mha_grads(q, k, v, ones, spec, softmax_scale=scale)
    _assert_close("out", out, want, dtype)
    for name, got, exp in (("dq", qd.grad, wq), ("dk", kd.grad, wk), ("dv", vd.grad, wv)):
        # gradients of a mean are ~1e-6: relative check
        assert got.dtype == dtype and ref.rel_l2(got.cpu(), exp) < (1e-4 if dtype == torch.float32 else 2e-2), name
    # Function-level entry point with a mask fn.
    o2 = flash_attention(qd, kd, vd, segment_ids=segs.cuda(), softmax_scale=scale,
                         mask_fn=ab.sliding_window_causal_mask(64))
    assert torch.equal(o2, out)
    # A dense bias of zeros goes through the dense-bias kernels and changes nothing.
    dense = ab.CompositeAttentionBias([
        ab.SlidingWindowAttentionBias(ab.sliding_window_causal_mask(64), sliding_window_size=64, **pos),
        ab.SegmentIdAttentionBias(segs.cuda()),
        ab.TensorAttentionBias(torch.zeros(1, 1, t, t, device="cuda")),
    ])
    impl = flash_attention_implementation("gpu", query=qd, key=kd, value=vd, bias=dense, softmax_scale=scale)
    assert impl is not None and isinstance(impl.fn, HipFlashAttention)
    o3 = impl.fn(dict(query=qd, key=kd, value=vd, bias=dense))
    assert ref.max_abs(o3.detach().cpu().float(), out.detach().cpu().float()) < 1e-2


@pytest.mark.parametrize("mask,window,ds_workspace", [("causal", None, False), ("causal", None, True),
                                                      ("sliding", 200, True)])
def test_forward_and_backward_replay_from_a_captured_graph(mask, window, ds_workspace):
    """Forward + backward enqueue kernels only, so they can be captured into a graph; every replay,
    with eager work between the replays, equals the eager result bit for bit.  Both backward paths
    (the dS-workspace one with its table of stored tiles as well)."""
    b, t, hq, hkv, d = 2, 512, 4, 2, 128
    q, k, v, do = (x.cuda() for x in _inputs(b, t, hq, hkv, d, torch.bfloat16))
    segs = ref.packed_segment_ids(4, b, t, max_docs=3).cuda()
    mk = ops.MASK_CAUSAL if mask == "causal" else ops.MASK_SLIDING_WINDOW
    kw = dict(softmax_scale=d ** -0.5, mask_kind=mk, sliding_window=window or 0, segment_ids=segs)
    out_e, lse_e = ops.flash_fwd(q, k, v, **kw)
    grads_e = ops.flash_bwd(q, k, v, out_e, lse_e, do, ds_workspace=ds_workspace, **kw)
    bufs = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v),
            ops.flash_bwd_buffers(q, k, v, mask_kind=mk, segment_ids=segs, ds_workspace=ds_workspace)[3])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g, lse_g = ops.flash_fwd(q, k, v, **kw)
        ops.flash_bwd(q, k, v, out_g, lse_g, do, buffers=bufs, ds_workspace=ds_workspace, **kw)
    for rep in range(3):
        for x in (out_g, lse_g, *bufs):
            x.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e) and torch.equal(lse_g, lse_e), rep
        assert all(torch.equal(g, e) for g, e in zip(bufs[:3], grads_e)), rep
        q.copy_(q.roll(1, dims=1))  # new inputs in the captured buffers
        out_e, lse_e = ops.flash_fwd(q, k, v, **kw)
        grads_e = ops.flash_bwd(q, k, v, out_e, lse_e, do, ds_workspace=ds_workspace, **kw)


# ----------------------------------------------------------------------------- logit sink, head dims


@pytest.mark.parametrize("b,t,hq,hkv,d,dtype,mask,window,seg", [
    (2, 256, 4, 2, 128, torch.bfloat16, "causal", None, False),
    (1, 512, 4, 4, 64, torch.bfloat16, "sliding", 100, True),
    (1, 384, 2, 1, 128, torch.bfloat16, "none", None, False),
    (1, 384, 4, 2, 128, torch.float16, "causal", None, True),
    (1, 256, 4, 2, 64, torch.float32, "causal", None, True),
    (1, 128, 2, 2, 128, torch.float32, "none", None, False),
])
def test_logit_sink_forward_and_backward(b, t, hq, hkv, d, dtype, mask, window, seg):
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype)
    segs = ref.packed_segment_ids(4, b, t, max_docs=4) if seg else None
    spec, kw = _mask_args(mask, window, segs)
    scale = d ** -0.5
    # Sinks from well below to well above the typical row maximum (logits are ~N(0, 1)).
    sink = torch.linspace(-3.0, 6.0, hq, dtype=torch.float32)
    want, want_lse = ref.reference_mha(q, k, v, spec, softmax_scale=scale, logit_sink=sink, return_lse=True)
    out, lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), softmax_scale=scale, logit_sink=sink.cuda(), **kw)
    _assert_close("out", out, want, dtype)
    assert ref.max_abs(lse.cpu(), want_lse) < (1e-5 if dtype == torch.float32 else 1e-3) * max(1.0, float(want_lse.abs().max()))
    # The sink must matter in this test: without it the output differs visibly.
    plain, _ = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), softmax_scale=scale, **kw)
    assert ref.max_abs(plain.cpu(), want) > 0.05
    wq, wk, wv, ws = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=scale, logit_sink=sink)
    dq, dk, dv, dsink = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), softmax_scale=scale,
                                     logit_sink=sink.cuda(), **kw)
    _assert_close("dq", dq, wq, dtype)
    _assert_close("dk", dk, wk, dtype)
    _assert_close("dv", dv, wv, dtype)
    assert dsink.dtype == torch.float32 and ref.rel_l2(dsink.cpu(), ws) < 1e-2, (dsink.cpu(), ws)
    # Extreme sinks: far below every logit it is invisible (bit-identical output), far above it
    # takes all the mass; neither produces non-finite values.
    low, _ = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), softmax_scale=scale,
                           logit_sink=torch.full((hq,), -1e4, device="cuda"), **kw)
    assert torch.equal(low, plain)
    high, high_lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), softmax_scale=scale,
                                   logit_sink=torch.full((hq,), 1e4, device="cuda"), **kw)
    assert high.abs().max() == 0 and torch.allclose(high_lse, torch.full_like(high_lse, 1e4))


def test_logit_sink_through_dispatch_with_autograd():
    b, t, hq, hkv, d = 1, 256, 4, 2, 64
    q, k, v, _ = _inputs(b, t, hq, hkv, d, torch.bfloat16)
    sink = torch.tensor([0.5, -1.0, 2.0, 0.0])
    qd, kd, vd = (x.cuda().requires_grad_(True) for x in (q, k, v))
    sd = sink.cuda().requires_grad_(True)
    pos = dict(target_positions=torch.arange(t)[None], source_positions=torch.arange(t)[None])
    bias = ab.CompositeAttentionBias([ab.CausalAttentionBias(**pos)])
    scale = d ** -0.5
    impl = flash_attention_implementation("gpu", query=qd, key=kd, value=vd, bias=bias, softmax_scale=scale,
                                          logit_sink=sd)
    assert impl is not None and isinstance(impl.fn, HipFlashAttention)
    out = impl.fn(dict(query=qd, key=kd, value=vd, bias=bias, logit_sink=sd))
    do = ref.normal_tensor(9, (b, t, hq, d), torch.bfloat16)
    (out.float() * do.cuda().float()).sum().backward()
    spec = ref.MaskSpec(causal=True)
    want = ref.reference_mha(q, k, v, spec, softmax_scale=scale, logit_sink=sink)
    wq, wk, wv, ws = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=scale, logit_sink=sink)
    _assert_close("out", out, want, torch.bfloat16)
    for name, got, exp in (("dq", qd.grad, wq), ("dk", kd.grad, wk), ("dv", vd.grad, wv)):
        _assert_close(name, got, exp, torch.bfloat16)
    assert sd.grad.shape == (hq,) and ref.rel_l2(sd.grad.cpu(), ws) < 1e-2


@pytest.mark.parametrize("d", [32, 72, 80, 96, 120])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_head_dims_between_the_compiled_widths(d, dtype, monkeypatch):
    """Any head dim up to 128 is accepted, as by the Pallas kernel (gpu_attention.py:172-176, :954).  In
    bf16 / f16 a multiple of 8 runs on the tensors as they are: no padded copy of q, k, v or dO is made
    (the padding helper must not be called), forward and both backward paths."""
    from axlearn_amd.flash_attention import hip_attention

    def no_padding(x, width):
        assert x.shape[-1] == width, "a padded copy was made"
        return x

    monkeypatch.setattr(hip_attention, "_pad_last", no_padding)
    b, t, hq, hkv = 2, 512, 4, 2
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype)
    scale = d ** -0.5
    segs = ref.packed_segment_ids(4, b, t, max_docs=3)
    pos = dict(target_positions=torch.arange(t)[None], source_positions=torch.arange(t)[None])
    for window, seg, ds in ((None, False, True), (None, False, False), (100, True, True), (100, True, False)):
        qd, kd, vd = (x.cuda().requires_grad_(True) for x in (q, k, v))
        mask = ab.CausalAttentionBias(**pos) if window is None else ab.SlidingWindowAttentionBias(
            ab.sliding_window_causal_mask(window), sliding_window_size=window, **pos)
        bias = ab.CompositeAttentionBias([mask] + ([ab.SegmentIdAttentionBias(segs.cuda())] if seg else []))
        fa = HipFlashAttention.default_config().set(softmax_scale=scale, bwd_ds_workspace=ds).instantiate()
        batch = dict(query=qd, key=kd, value=vd, bias=bias)
        assert fa.is_supported(batch, kv_cache_type=None)
        out = fa(batch)
        assert out.shape == (b, t, hq, d)
        (out.float() * do.cuda().float()).sum().backward()
        spec = ref.MaskSpec(causal=window is None, sliding_window=window, segment_ids=segs if seg else None)
        want = ref.reference_mha(q, k, v, spec, softmax_scale=scale)
        wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=scale)
        _assert_close("out", out, want, dtype)
        for name, got, exp in (("dq", qd.grad, wq), ("dk", kd.grad, wk), ("dv", vd.grad, wv)):
            assert got.shape == exp.shape and got.is_contiguous()
            _assert_close(name, got, exp, dtype)


def test_head_dim_columns_past_the_end_are_never_used():
    """head_dim 72 as a view of wider tensors whose other columns hold NaN: neither the forward nor the
    backward lets one of them into a result (the tile loads stay inside the 72 columns)."""
    b, t, hq, hkv, d, wide = 1, 256, 4, 2, 72, 128
    q, k, v, do = _inputs(b, t, hq, hkv, d, torch.bfloat16)

    def widen(x):
        w = torch.full(x.shape[:-1] + (wide,), float("nan"), dtype=x.dtype, device="cuda")
        w[..., :d] = x.cuda()
        return w[..., :d]

    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_CAUSAL)
    out, lse = ops.flash_fwd(widen(q), widen(k), widen(v), **kw)
    base, base_lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), **kw)
    assert torch.equal(out, base) and torch.equal(lse, base_lse)
    for ds in (False, True):
        got = ops.flash_bwd(widen(q), widen(k), widen(v), widen(out.cpu()), lse, widen(do), ds_workspace=ds, **kw)
        want = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), base, base_lse, do.cuda(), ds_workspace=ds, **kw)
        for x, y in zip(got, want):
            assert torch.isfinite(x.float()).all() and torch.equal(x, y)


@pytest.mark.parametrize("d,dtype,hq,hkv", [(36, torch.bfloat16, 4, 2), (80, torch.float32, 4, 2), (72, torch.bfloat16, 1, 1),
                                             (8, torch.bfloat16, 4, 2)])
def test_head_dims_that_take_the_padded_path(d, dtype, hq, hkv):
    """What the kernels do not take as it is - a head dim that is not a multiple of 8, float32, rows
    closer together than the compiled width - is zero-padded by the host mirror and sliced."""
    b, t = 1, 256
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype)
    qd, kd, vd = (x.cuda().requires_grad_(True) for x in (q, k, v))
    scale = d ** -0.5
    out = flash_attention(qd, kd, vd, softmax_scale=scale, mask_fn=ab.causal_mask)
    assert out.shape == (b, t, hq, d)
    (out.float() * do.cuda().float()).sum().backward()
    spec = ref.MaskSpec(causal=True)
    want = ref.reference_mha(q, k, v, spec, softmax_scale=scale)
    wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=scale)
    _assert_close("out", out, want, dtype)
    for name, got, exp in (("dq", qd.grad, wq), ("dk", kd.grad, wk), ("dv", vd.grad, wv)):
        assert got.shape == exp.shape
        _assert_close(name, got, exp, dtype)


# ----------------------------------------------------------------------------- dense bias, dropout


def _dense_bias(seed, shape, dtype):
    # Values of a few units, as relative-position biases have; a band of -1e15 entries as masks have.
    g = torch.Generator().manual_seed(seed)
    bias = torch.randn(shape, generator=g) * 2.0
    t, s = shape[-2:]
    band = (torch.arange(t)[:, None] - torch.arange(s)[None, :]).abs() % 37 == 5
    return torch.where(band, torch.tensor(ref.NEG_INF), bias).to(dtype)


AUX_CASES = [
    # b, t, s, hq, hkv, d, dtype, mask, window, seg, bias shape (None = none), bias dtype, dropout rate
    (2, 256, 256, 4, 2, 128, torch.bfloat16, "none", None, False, "bh", torch.bfloat16, 0.0),
    (2, 256, 256, 4, 2, 128, torch.bfloat16, "causal", None, True, "1h", torch.float32, 0.0),
    (1, 384, 384, 4, 4, 64, torch.bfloat16, "sliding", 100, False, "11", torch.float32, 0.0),
    (2, 256, 256, 4, 2, 128, torch.bfloat16, "causal", None, False, None, None, 0.3),
    (1, 384, 384, 6, 2, 64, torch.bfloat16, "none", None, True, None, None, 0.1),
    (2, 256, 384, 4, 1, 128, torch.bfloat16, "none", None, False, "b1", torch.bfloat16, 0.2),
    (1, 256, 256, 8, 2, 64, torch.bfloat16, "causal", None, True, "bh", torch.float32, 0.5),
    (1, 256, 256, 2, 2, 64, torch.float32, "causal", None, False, "bh", torch.float32, 0.25),
    (1, 128, 256, 2, 1, 128, torch.float32, "none", None, False, "1h", torch.bfloat16, 0.0),
    # float16 q/k/v: a float16 bias is handed over as float32 by the wrapper
    (2, 256, 256, 4, 2, 128, torch.float16, "causal", None, True, "1h", torch.float16, 0.0),
    (1, 256, 384, 4, 1, 64, torch.float16, "none", None, False, "bh", torch.float32, 0.2),
]


@pytest.mark.parametrize("b,t,s,hq,hkv,d,dtype,mask,window,seg,bias_kind,bias_dtype,rate", AUX_CASES)
def test_dense_bias_and_dropout_forward_and_backward(b, t, s, hq, hkv, d, dtype, mask, window, seg, bias_kind,
                                                     bias_dtype, rate):
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype, s=s)
    segs = ref.packed_segment_ids(4, b, t, max_docs=4) if seg else None
    spec, kw = _mask_args(mask, window, segs)
    bias = None
    if bias_kind is not None:
        shape = (b if bias_kind[0] == "b" else 1, hq if bias_kind[1] == "h" else 1, t, s)
        bias = _dense_bias(11, shape, bias_dtype)
        spec.dense_bias = bias.float()
    drop = None
    if rate > 0:
        drop = torch.rand((b, hq, t, s), generator=torch.Generator().manual_seed(12)) < rate
    scale = d ** -0.5
    okw = dict(softmax_scale=scale, dropout_mask=drop, dropout_rate=rate)
    want, want_lse = ref.reference_mha(q, k, v, spec, return_lse=True, **okw)
    gkw = dict(softmax_scale=scale, bias=None if bias is None else bias.cuda(),
               dropout_mask=None if drop is None else drop.cuda(), dropout_rate=rate, **kw)
    out, lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), **gkw)
    _assert_close("out", out, want, dtype)
    assert ref.max_abs(lse.cpu(), want_lse) < (1e-5 if dtype == torch.float32 else 1e-3) * max(1.0, float(want_lse.abs().max()))
    # The optional inputs must matter in this test.
    plain, _ = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), softmax_scale=scale, **kw)
    assert ref.max_abs(plain.cpu(), want) > 0.05
    wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, **okw)
    dq, dk, dv = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), **gkw)
    _assert_close("dq", dq, wq, dtype)
    _assert_close("dk", dk, wk, dtype)
    _assert_close("dv", dv, wv, dtype)


def test_dropout_mask_is_applied_exactly():
    # Poison: a value row of 1e30 behind a dropped probability must leave no trace; dropping
    # everything gives exact zeros with an untouched lse; dropping nothing at rate r is a rescale.
    b, t, hq, hkv, d = 1, 256, 2, 1, 128
    q, k, v, _ = _inputs(b, t, hq, hkv, d, torch.bfloat16)
    drop = torch.zeros((b, hq, t, t), dtype=torch.bool)
    drop[:, :, :, 77] = True
    vp = v.clone()
    vp[:, 77] = 1e30
    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_CAUSAL, dropout_rate=0.5)
    got, lse = ops.flash_fwd(q.cuda(), k.cuda(), vp.cuda(), dropout_mask=drop.cuda(), **kw)
    want, _ = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), dropout_mask=drop.cuda(), **kw)
    assert torch.isfinite(got.float()).all() and torch.equal(got, want)
    base, base_lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), softmax_scale=d ** -0.5, mask_kind=ops.MASK_CAUSAL)
    assert torch.equal(lse, base_lse)
    zero, zlse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), dropout_mask=torch.ones_like(drop).cuda(), **kw)
    assert zero.abs().max() == 0 and torch.equal(zlse, base_lse)
    none, _ = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), dropout_mask=torch.zeros_like(drop).cuda(), **kw)
    assert ref.max_abs(none.cpu().float(), base.cpu().float() * 2) < 2e-2
    # A bias of -1e15 on a column acts as a mask for that column (poison again), in fwd and bwd.
    bias = torch.zeros((1, 1, t, t))
    bias[..., 77] = ref.NEG_INF
    got, lse = ops.flash_fwd(q.cuda(), k.cuda(), vp.cuda(), bias=bias.cuda(), softmax_scale=d ** -0.5)
    assert torch.isfinite(got.float()).all()
    do = ref.normal_tensor(5, (b, t, hq, d), torch.bfloat16).cuda()
    dq, dk, dv = ops.flash_bwd(q.cuda(), k.cuda(), vp.cuda(), got, lse, do, bias=bias.cuda(), softmax_scale=d ** -0.5)
    assert dk[:, 77].abs().max() == 0 and dv[:, 77].abs().max() == 0
    assert all(torch.isfinite(x.float()).all() for x in (dq, dk, dv))


def test_arbitrary_mask_fn_explicit_bias_and_dropout_through_dispatch():
    b, t, hq, hkv, d = 2, 256, 4, 2, 64
    q, k, v, do = _inputs(b, t, hq, hkv, d, torch.bfloat16)
    qd, kd, vd = (x.cuda().requires_grad_(True) for x in (q, k, v))
    scale = d ** -0.5

    def strided_causal(qp, kp):  # not a mask the kernels have a closed form for
        return (qp >= kp) & ((qp - kp) % 3 != 1)

    rel = _dense_bias(21, (1, hq, t, t), torch.float32)
    rel = torch.where(rel < -1e14, torch.zeros(()), rel)
    pos = dict(target_positions=torch.arange(t)[None].cuda(), source_positions=torch.arange(t)[None].cuda())
    bias = ab.CompositeAttentionBias([
        ab.MaskFnAttentionBias(strided_causal, **pos),
        ab.TensorAttentionBias(rel.cuda()),
    ])
    rate = 0.2
    impl = flash_attention_implementation("gpu", query=qd, key=kd, value=vd, bias=bias, softmax_scale=scale,
                                          dropout_rate=rate)
    assert impl is None  # dropout without a prng_key cannot be served
    fa = HipFlashAttention.default_config().set(softmax_scale=scale, dropout_rate=rate).instantiate()
    batch = dict(query=qd, key=kd, value=vd, bias=bias, prng_key=1234)
    assert fa.is_supported(batch, kv_cache_type=None)
    out = fa(batch)
    (out.float() * do.cuda().float()).sum().backward()
    from axlearn_amd.flash_attention.hip_attention import get_dropout_mask
    drop = get_dropout_mask((b, hq, t, t), prng_key=1234, rate=rate, device="cuda").cpu()
    assert 0.15 < drop.float().mean() < 0.25
    keep = strided_causal(torch.arange(t)[:, None], torch.arange(t)[None, :])
    spec = ref.MaskSpec(dense_bias=rel + torch.where(keep, 0.0, ref.NEG_INF)[None, None])
    okw = dict(softmax_scale=scale, dropout_mask=drop, dropout_rate=rate)
    want = ref.reference_mha(q, k, v, spec, **okw)
    wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, **okw)
    _assert_close("out", out, want, torch.bfloat16)
    for name, got, exp in (("dq", qd.grad, wq), ("dk", kd.grad, wk), ("dv", vd.grad, wv)):
        _assert_close(name, got, exp, torch.bfloat16)
    # Function-level entry point: same mask fn, same key, same result.
    o2 = flash_attention(qd, kd, vd, bias=rel.cuda(), softmax_scale=scale, mask_fn=strided_causal,
                         dropout_rate=rate, prng_key=1234)
    assert torch.equal(o2, out)


# ----------------------------------------------------------------------------- incremental prefill, remat


@pytest.mark.parametrize("bias_type", ["causal", "sliding"])
@pytest.mark.parametrize("prefix_len", [[64] * 4, [32, 40, 48, 56]])
@pytest.mark.parametrize("suffix_len", [16, 64, 160])
def test_incremental_prefill_matches_full_forward(bias_type, prefix_len, suffix_len):
    # The reference's test of the same name (utils_test.py:361-478): each sequence appends a chunk of
    # queries after a prefix of its own length; the result must equal those rows of a full forward.
    from axlearn_amd.kv_cache import KVCache

    b, hq, hkv, d, kv_len = 4, 4, 2, 64, 256
    q, k, v, _ = _inputs(b, kv_len, hq, hkv, d, torch.bfloat16)
    prefix = torch.tensor(prefix_len)
    window = 4

    def make_bias(target_positions):
        pos = dict(target_positions=target_positions.cuda(), source_positions=torch.arange(kv_len)[None].cuda())
        if bias_type == "causal":
            return ab.CompositeAttentionBias([ab.CausalAttentionBias(**pos)])
        return ab.CompositeAttentionBias([
            ab.SlidingWindowAttentionBias(ab.sliding_window_causal_mask(window), sliding_window_size=window, **pos)])

    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    fwd_bias = make_bias(torch.arange(kv_len)[None].expand(b, kv_len))
    fwd = flash_attention_implementation("gpu", query=qc, key=kc, value=vc, bias=fwd_bias)
    fwd_out = fwd.fn(dict(query=qc, key=kc, value=vc, bias=fwd_bias))
    incr_positions = torch.arange(suffix_len)[None] + prefix[:, None]
    incr_bias = make_bias(incr_positions)
    rows = incr_positions.cuda()[:, :, None, None].expand(b, suffix_len, hq, d)
    suffix_q = torch.gather(qc, 1, rows)
    incr = flash_attention_implementation("gpu", query=suffix_q, key=kc, value=vc, bias=incr_bias, kv_cache_type=KVCache)
    assert incr is not None and isinstance(incr.fn, HipFlashAttention)
    incr_out = incr.fn(dict(query=suffix_q, key=kc, value=vc, bias=incr_bias))
    assert incr_out.shape == (b, suffix_len, hq, d)
    assert torch.equal(incr_out, torch.gather(fwd_out, 1, rows))
    # And against the oracle evaluated with the per-batch positions.
    spec = ref.MaskSpec(causal=bias_type == "causal", sliding_window=window if bias_type == "sliding" else None,
                        target_positions=incr_positions, source_positions=torch.arange(kv_len)[None])
    want = ref.reference_mha(suffix_q.cpu(), k, v, spec)
    _assert_close("incremental", incr_out, want, torch.bfloat16)


def test_backward_without_saved_residuals_is_bit_identical():
    b, t, hq, hkv, d = 2, 256, 4, 2, 128
    q, k, v, do = _inputs(b, t, hq, hkv, d, torch.bfloat16)
    pos = dict(target_positions=torch.arange(t)[None], source_positions=torch.arange(t)[None])
    bias = ab.CompositeAttentionBias([ab.CausalAttentionBias(**pos)])
    sink = torch.tensor([0.1, -0.4, 1.0, 0.0], device="cuda")
    grads = []
    for cfg in (dict(), dict(save_residuals=False), dict(backend_overrides=dict(save_residuals=False))):
        qd, kd, vd = (x.cuda().requires_grad_(True) for x in (q, k, v))
        sd = sink.clone().requires_grad_(True)
        fa = HipFlashAttention.default_config().set(softmax_scale=d ** -0.5, **cfg).instantiate()
        batch = dict(query=qd, key=kd, value=vd, bias=bias, logit_sink=sd)
        assert fa.is_supported(batch, kv_cache_type=None)
        out = fa(batch)
        saved = [x for x in out.grad_fn.saved_tensors if x is not None]
        assert len(saved) == (6 if not cfg else 4)  # q, k, v, sink (+ out, lse)
        (out.float() * do.cuda().float()).sum().backward()
        grads.append((out.detach(), qd.grad, kd.grad, vd.grad, sd.grad))
    for other in grads[1:]:
        for x, y in zip(grads[0], other):
            assert torch.equal(x, y)


def test_ds_workspace_backward_through_the_plugin_config():
    """`bwd_ds_workspace` (config field or backend override) reaches the backward: dv is bit-identical
    to the recomputing path's, dq and dk agree to summation order, and the gradients match the kernel
    called directly with the flag.  Left at its default (None) the choice goes by size: the dS
    workspace where it fits `bwd_workspace_limit_bytes` (default a sixteenth of the device's memory),
    the recomputing pair where it does not."""
    b, t, hq, hkv, d = 2, 512, 4, 2, 128
    q, k, v, do = _inputs(b, t, hq, hkv, d, torch.bfloat16)
    pos = dict(target_positions=torch.arange(t)[None], source_positions=torch.arange(t)[None])
    bias = ab.CompositeAttentionBias([
        ab.SlidingWindowAttentionBias(ab.sliding_window_causal_mask(100), sliding_window_size=100, **pos)])
    grads = []
    need, plain = ops.flash_bwd_ds_workspace_bytes(q.cuda(), k.cuda(), mask_kind=ops.MASK_SLIDING_WINDOW)
    assert plain < need < ops.default_bwd_workspace_limit(torch.device("cuda:0"))
    for cfg in (dict(bwd_ds_workspace=False), dict(bwd_ds_workspace=True),
                dict(backend_overrides=dict(bwd_ds_workspace=True)),
                dict(),                                                # fits the default limit: dS workspace
                dict(bwd_workspace_limit_bytes=need),                  # just fits
                dict(bwd_workspace_limit_bytes=need - 1),              # does not: recomputing pair
                dict(backend_overrides=dict(bwd_workspace_limit_bytes=plain))):
        qd, kd, vd = (x.cuda().requires_grad_(True) for x in (q, k, v))
        fa = HipFlashAttention.default_config().set(softmax_scale=d ** -0.5, **cfg).instantiate()
        out = fa(dict(query=qd, key=kd, value=vd, bias=bias))
        (out.float() * do.cuda().float()).sum().backward()
        grads.append((out.detach(), qd.grad, kd.grad, vd.grad))
    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_SLIDING_WINDOW, sliding_window=100)
    out, lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), **kw)
    direct = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), ds_workspace=True, **kw)
    for g in grads[1:5]:
        assert torch.equal(g[0], grads[0][0]) and torch.equal(g[3], grads[0][3])
        assert all(torch.equal(x, y) for x, y in zip(g[1:], direct))
        assert not torch.equal(g[1], grads[0][1])  # a different dq kernel ran
        assert ref.rel_l2(g[1].cpu(), grads[0][1].cpu().float()) < 1e-4
    for g in grads[5:]:
        assert all(torch.equal(x, y) for x, y in zip(g, grads[0]))


def test_plugin_takes_the_ds_workspace_in_slices_when_the_whole_does_not_fit():
    """A limit just below the whole dS workspace, on a shape whose slices still fill the GPU: the default
    configuration keeps the dS of 7 of the 8 kv heads at a time (then the last one), and the gradients are
    bit-identical to the kernel called directly with the whole workspace; the same through
    `ops.flash_bwd(ds_workspace=None, ds_workspace_limit=...)`."""
    b, t, hq, hkv, d = 8, 2048, 8, 8, 64
    q, k, v, do = (x.cuda() for x in _inputs(b, t, hq, hkv, d, torch.bfloat16))
    full, plain = ops.flash_bwd_ds_workspace_bytes(q, k, mask_kind=ops.MASK_CAUSAL)
    assert ops.select_ds_slice(q, k, mask_kind=ops.MASK_CAUSAL, limit=full - 1) == (True, hkv - 1)
    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_CAUSAL)
    out, lse = ops.flash_fwd(q, k, v, **kw)
    direct = ops.flash_bwd(q, k, v, out, lse, do, ds_workspace=True, **kw)
    auto = ops.flash_bwd(q, k, v, out, lse, do, ds_workspace=None, ds_workspace_limit=full - 1, **kw)
    assert all(torch.equal(x, y) for x, y in zip(auto, direct))
    pos = dict(target_positions=torch.arange(t)[None], source_positions=torch.arange(t)[None])
    bias = ab.CompositeAttentionBias([ab.CausalAttentionBias(**pos)])
    qd, kd, vd = (x.clone().requires_grad_(True) for x in (q, k, v))
    fa = HipFlashAttention.default_config().set(softmax_scale=d ** -0.5, bwd_workspace_limit_bytes=full - 1).instantiate()
    res = fa(dict(query=qd, key=kd, value=vd, bias=bias))
    grads = torch.autograd.grad(res, (qd, kd, vd), do)
    assert torch.equal(res, out) and all(torch.equal(x, y) for x, y in zip(grads, direct))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rows_without_a_visible_key(dtype):
    """Causal rows at negative positions see no key: out = 0, lse = -inf, and the backward leaves dq of
    those rows at zero and every gradient finite; the other rows match the oracle on the sub-problem
    without the empty rows."""
    b, t, hq, hkv, d, off = 2, 256, 4, 2, 128, -100
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype)
    kw = dict(softmax_scale=d ** -0.5, mask_kind=ops.MASK_CAUSAL, q_pos_offset=off)
    out, lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), **kw)
    dq, dk, dv = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), **kw)
    e = -off
    assert (out[:, :e] == 0).all() and torch.isinf(lse[:, :, :e]).all() and (lse[:, :, :e] < 0).all()
    assert (dq[:, :e] == 0).all()
    for x in (out, dq, dk, dv):
        assert torch.isfinite(x.float()).all()
    assert torch.isfinite(lse[:, :, e:]).all()
    spec = ref.MaskSpec(causal=True, target_positions=torch.arange(t - e)[None], source_positions=torch.arange(t)[None])
    want = ref.reference_mha(q[:, e:], k, v, spec, softmax_scale=d ** -0.5)
    wq, wk, wv = ref.reference_mha_grads(q[:, e:], k, v, do[:, e:], spec, softmax_scale=d ** -0.5)
    _assert_close("out", out[:, e:], want, dtype)
    _assert_close("dq", dq[:, e:], wq, dtype)
    _assert_close("dk", dk, wk, dtype)
    _assert_close("dv", dv, wv, dtype)


@pytest.mark.parametrize("b,t,hq,hkv,d,dtype", [
    (1, 256, 4, 2, 128, torch.bfloat16), (2, 512, 8, 2, 128, torch.bfloat16), (1, 1024, 4, 1, 64, torch.bfloat16),
    (2, 384, 6, 6, 128, torch.float16), (8, 1152, 8, 2, 128, torch.bfloat16), (3, 640, 10, 5, 64, torch.float16),
])
def test_ds_workspace_backward_matches_oracle(b, t, hq, hkv, d, dtype):
    """The backward that keeps dS in the workspace (AXL_BWD_DS_WORKSPACE): dq, dk, dv against the
    oracle, dv bit-identical to the recompute path's (same arithmetic up to dS), also with a logit sink."""
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype)
    spec = ref.MaskSpec(causal=True)
    scale = d ** -0.5
    sink = torch.linspace(-1.0, 1.0, hq)
    for sk in (None, sink):
        kw = dict(softmax_scale=scale, mask_kind=ops.MASK_CAUSAL, logit_sink=None if sk is None else sk.cuda())
        out, lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), **kw)
        got = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), ds_workspace=True, **kw)
        base = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), **kw)
        want = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=scale, logit_sink=sk)
        for name, x, w in zip(("dq", "dk", "dv"), got, want):
            _assert_close(name, x, w, dtype)
        assert torch.equal(got[2], base[2])
        if sk is not None:
            assert ref.max_abs(got[3].cpu(), want[3]) <= 2e-2 * max(1.0, float(want[3].abs().max()))
    # the flag is ignored where the path does not apply (here: no mask)
    kw = dict(softmax_scale=scale, mask_kind=ops.MASK_NONE)
    out, lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), **kw)
    a = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), ds_workspace=True, **kw)
    c = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), **kw)
    assert all(torch.equal(x, y) for x, y in zip(a, c))


@pytest.mark.parametrize("b,t,hq,hkv,d,dtype,mask,window,seg", [
    (1, 512, 4, 2, 128, torch.bfloat16, "causal", None, "packed"),
    (2, 512, 4, 2, 128, torch.bfloat16, "sliding", 100, None),
    (2, 1024, 8, 2, 128, torch.bfloat16, "sliding", 300, "packed"),
    (1, 1024, 4, 1, 64, torch.bfloat16, "sliding", 200, "packed"),
    (3, 640, 10, 5, 64, torch.float16, "sliding", 31, "packed"),
    # ids that come back later in the row: the key blocks that hold dS for a query tile are then not one run
    (2, 768, 6, 6, 128, torch.float16, "causal", None, "unsorted"),
    # head_dim 128 with a length that is not a multiple of 256: the flag falls back to the recomputing path
    (1, 384, 4, 4, 128, torch.bfloat16, "sliding", 64, "packed"),
])
def test_ds_workspace_backward_under_window_and_segments(b, t, hq, hkv, d, dtype, mask, window, seg):
    """AXL_BWD_DS_WORKSPACE under a sliding window and / or segment ids: the dK/dV kernel records which
    query tiles each key block stored dS for and the streaming dQ kernel reads only those.  Against the
    oracle, and dv bit-identical to the recomputing path's."""
    q, k, v, do = _inputs(b, t, hq, hkv, d, dtype)
    segs = None
    if seg is not None:
        segs = ref.packed_segment_ids(4, b, t, max_docs=4)
        if seg == "unsorted":
            segs = (segs * 7) % 5 + 1
    spec, kw = _mask_args(mask, window, segs)
    scale = d ** -0.5
    out, lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), softmax_scale=scale, **kw)
    bufs = ops.flash_bwd_buffers(q.cuda(), k.cuda(), v.cuda(), mask_kind=kw["mask_kind"], ds_workspace=True,
                                 segment_ids=kw["segment_ids"])
    bufs[3].fill_(0xff)   # blocks nobody stores must not be read: as NaN patterns they would show
    got = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), softmax_scale=scale, ds_workspace=True,
                        buffers=bufs, **kw)
    base = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), softmax_scale=scale, **kw)
    want = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=scale)
    for name, x, w in zip(("dq", "dk", "dv"), got, want):
        _assert_close(name, x, w, dtype)
    assert torch.equal(got[2], base[2])
    assert ref.rel_l2(got[0].cpu(), base[0].cpu().float()) < 1e-4


@pytest.mark.parametrize("seed", range(10))
def test_ds_workspace_sweep_against_the_recomputing_path(seed):
    """Seeded sweep at sizes the oracle would take long for: lengths up to 4096, batch x kv heads spread
    over the XCDs or not, windows from a few keys to the whole row, 1..6 documents per row.  The two
    backward paths share everything up to dS, so dv is bit-identical, dk differs only through delta's
    summation order and dq through its own; the workspace starts out as NaN patterns."""
    rng = np.random.default_rng(4000 + seed)
    d = int(rng.choice([64, 128]))
    dtype = [torch.bfloat16, torch.float16][int(rng.integers(0, 2))]
    hkv = int(rng.choice([1, 2, 4, 8]))
    hq = hkv * int(rng.choice([1, 2, 4]))
    b = int(rng.choice([1, 2, 4]))
    t = 256 * int(rng.integers(1, 17))
    kind = str(rng.choice(["causal", "sliding"]))
    window = int(rng.choice([7, 100, t // 3, t - 1, 2 * t])) if kind == "sliding" else None
    packed = bool(rng.integers(0, 2))
    q, k, v, do = (x.cuda() for x in _inputs(b, t, hq, hkv, d, dtype))
    segs = ref.packed_segment_ids(seed, b, t).cuda() if packed else None
    mk = ops.MASK_CAUSAL if kind == "causal" else ops.MASK_SLIDING_WINDOW
    kw = dict(mask_kind=mk, sliding_window=window or 0, softmax_scale=d ** -0.5, segment_ids=segs)
    case = f"b={b} t={t} hq={hq} hkv={hkv} d={d} {dtype} {kind} window={window} packed={packed}"
    out, lse = ops.flash_fwd(q, k, v, **kw)
    bufs = ops.flash_bwd_buffers(q, k, v, mask_kind=mk, ds_workspace=True, segment_ids=segs)
    bufs[3].fill_(0xff)
    dq, dk, dv = ops.flash_bwd(q, k, v, out, lse, do, ds_workspace=True, buffers=bufs, **kw)
    bq, bk, bv = ops.flash_bwd(q, k, v, out, lse, do, **kw)
    assert torch.equal(dv, bv), case
    for name, x, y in (("dq", dq, bq), ("dk", dk, bk)):
        assert torch.isfinite(x.float()).all(), f"{name} {case}"
        assert ref.rel_l2(x.cpu(), y.cpu().float()) < 1e-4, f"{name} {case}: {ref.rel_l2(x.cpu(), y.cpu().float()):.3e}"


@pytest.mark.parametrize("b,t,hq,hkv,d,kind,window,packed", [
    (2, 512, 8, 4, 128, "causal", None, False),
    (1, 768, 6, 3, 64, "causal", None, True),
    (2, 512, 4, 4, 128, "sliding", 200, True),
    (1, 1024, 10, 5, 64, "sliding", 77, False),
])
def test_ds_workspace_in_slices_of_kv_heads_is_bit_identical(b, t, hq, hkv, d, kind, window, packed):
    """AXL_BWD_DS_SLICE_KV_HEADS: the workspace holds the dS of n kv heads at a time and the dK/dV and dQ
    kernels run slice after slice (every n from 1 to hkv - 1, so uneven last slices too).  A slice's
    kernels do what the whole launch does for those heads, so dq, dk and dv are bit-identical to the
    unsliced path; the workspace shrinks by the dS of the heads left out; the dK/dV phase without the
    dQ phase is refused (the next slice would overwrite what it left); the automatic choice takes the
    largest slice that fits its limit, or the recomputing pair when a slice would not fill the GPU."""
    q, k, v, do = (x.cuda() for x in _inputs(b, t, hq, hkv, d, torch.bfloat16))
    segs = ref.packed_segment_ids(7, b, t).cuda() if packed else None
    mk = ops.MASK_CAUSAL if kind == "causal" else ops.MASK_SLIDING_WINDOW
    kw = dict(mask_kind=mk, sliding_window=window or 0, softmax_scale=d ** -0.5, segment_ids=segs)
    out, lse = ops.flash_fwd(q, k, v, **kw)
    whole = ops.flash_bwd(q, k, v, out, lse, do, ds_workspace=True, **kw)
    full, plain = ops.flash_bwd_ds_workspace_bytes(q, k, mask_kind=mk, segment_ids=segs)
    for n in range(1, hkv):
        need, _ = ops.flash_bwd_ds_workspace_bytes(q, k, mask_kind=mk, segment_ids=segs, ds_slice_kv_heads=n)
        assert abs((need - plain) - (full - plain) * n // hkv) <= 512, n   # dS of n heads (+ the table of stored tiles)
        bufs = ops.flash_bwd_buffers(q, k, v, mask_kind=mk, ds_workspace=True, segment_ids=segs, ds_slice_kv_heads=n)
        assert bufs[3].numel() == max(need, 256)
        bufs[3].fill_(0xff)
        got = ops.flash_bwd(q, k, v, out, lse, do, ds_workspace=True, ds_slice_kv_heads=n, buffers=bufs, **kw)
        for name, x, y in zip(("dq", "dk", "dv"), got, whole):
            assert torch.equal(x, y), f"{name} with slices of {n}"
        with pytest.raises(ops.AxlError) as err:
            ops.flash_bwd(q, k, v, out, lse, do, ds_workspace=True, ds_slice_kv_heads=n, buffers=bufs, phases=2, **kw)
        assert err.value.code == _lib.AXL_ERR_UNSUPPORTED
    # the automatic choice: whole where it fits; slices where they fit and fill the CUs; else recompute
    assert ops.select_ds_slice(q, k, mask_kind=mk, segment_ids=segs, limit=full) == (True, 0)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    per_head = b * (t // 128) // (2 if kind == "causal" else 1)
    use, n = ops.select_ds_slice(q, k, mask_kind=mk, segment_ids=segs, limit=full - 1)
    assert (use, n) == ((True, hkv - 1) if (hkv - 1) * per_head >= cus else (False, 0))
    assert ops.select_ds_slice(q, k, mask_kind=mk, segment_ids=segs, limit=plain) == (False, 0)


def test_layer_compute_attention_end_to_end():
    """The layer-level calling sequence (layer.py:218-376) over the HIP kernels: bias cast to the query
    dtype, softmax_scale 1.0 by default with the scale folded into q beforehand, `(context, probs)` with
    probs a shape without contents, prefill and both decode paths, autograd through the context."""
    from axlearn_amd.flash_attention.layer import FlashAttention
    from axlearn_amd.kv_cache import KVCache, PagedKVCache

    b, t, hq, hkv, d = 2, 256, 8, 2, 128
    q, k, v, do = _inputs(b, t, hq, hkv, d, torch.bfloat16)
    scale = d ** -0.5
    q_scaled = (q.float() * scale).to(torch.bfloat16)   # `scale_query` happens before the layer calls the kernels
    pos = dict(target_positions=torch.arange(t)[None], source_positions=torch.arange(t)[None])
    bias = ab.CompositeAttentionBias([ab.CausalAttentionBias(**pos)])
    layer = FlashAttention.default_config().instantiate()
    qd, kd, vd = (x.cuda().requires_grad_(True) for x in (q_scaled, k, v))
    ctx, probs = layer.compute_attention(q_proj=qd, k_proj=kd, v_proj=vd, attention_logit_biases=bias)
    assert probs.device.type == "meta" and tuple(probs.shape) == (b, hq, t, t)
    spec = ref.MaskSpec(causal=True)
    want = ref.reference_mha(q_scaled, k, v, spec, softmax_scale=1.0)
    _assert_close("context", ctx, want, torch.bfloat16)
    ctx.backward(do.cuda())
    wq, wk, wv = ref.reference_mha_grads(q_scaled, k, v, do, spec, softmax_scale=1.0)
    _assert_close("dq", qd.grad, wq, torch.bfloat16)
    _assert_close("dk", kd.grad, wk, torch.bfloat16)
    _assert_close("dv", vd.grad, wv, torch.bfloat16)
    # an explicit softmax_scale is passed through
    layer2 = FlashAttention.default_config().set(softmax_scale=scale).instantiate()
    ctx2, _ = layer2.compute_attention(q_proj=q.cuda(), k_proj=k.cuda(), v_proj=v.cuda(), attention_logit_biases=bias)
    _assert_close("context (scale in the kernel)", ctx2, ref.reference_mha(q, k, v, spec, softmax_scale=scale), torch.bfloat16)
    # decode: contiguous cache, then paged pools with page_indices
    qq, kp, vp, tables, lengths = ref.paged_inputs(5, batch=3, num_heads=hq, num_kv_heads=hkv, head_dim=d, page_size=16,
                                                   pages_per_seq=8, min_len=10, max_len=128)
    dbias = ab.CompositeAttentionBias([ab.CausalAttentionBias(
        target_positions=(lengths.long() - 1)[:, None], source_positions=torch.arange(128)[None])])
    want_d = ref.reference_decode(qq, kp, vp, lengths, softmax_scale=1.0, page_tables=tables)
    got_p, probs_p = layer.compute_attention(q_proj=qq.cuda(), k_proj=kp.cuda(), v_proj=vp.cuda(),
                                             attention_logit_biases=dbias, page_indices=tables.cuda(),
                                             kv_cache_type=PagedKVCache)
    assert tuple(probs_p.shape) == (3, hq, 1, 128)
    _assert_close("paged decode", got_p, want_d, torch.bfloat16)
    kk, vv = ref.reconstruct_kv(tables, kp), ref.reconstruct_kv(tables, vp)
    got_c, _ = layer.compute_attention(q_proj=qq.cuda(), k_proj=kk.cuda(), v_proj=vv.cuda(),
                                       attention_logit_biases=dbias, kv_cache_type=KVCache)
    _assert_close("contiguous decode", got_c, want_d, torch.bfloat16)


# ----------------------------------------------------------------------------- BASELINE sizes


def _rel_ok(got, want):
    """The relative-L2 arm of the bf16 bar alone: on late rows of a long sequence outputs and
    gradients are small (rms ~ 0.03), so the max-abs arm would pass errors of tens of percent."""
    return ref.rel_l2(got, want) <= BF16_REL_L2


def _sampled_fwd_bwd_check(B, T, Hq, Hkv, D, mask, window, seg, samples, dq_rows, key_blocks=(), ds_workspace=False):
    """Full-size run on the GPU; the oracle checks sampled (batch, kv head) groups on query-row
    windows (a causal row only needs the keys before it) and on key blocks (dK/dV of a key block
    only needs the query rows that can see it, each with all the keys it normalises over), and
    size-independent identities check the rest: sum_s dV == sum_t dO and sum_s dK == 0 for every
    (batch, kv head)."""
    dev = "cuda"
    gen = torch.Generator(device=dev).manual_seed(0)
    mk = lambda h: torch.randn((B, T, h, D), device=dev, generator=gen).to(torch.bfloat16)
    q, k, v, do = mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)
    segs = ref.packed_segment_ids(4, B, T) if seg else None
    spec_kw = dict(causal=mask == "causal", sliding_window=window if mask == "sliding" else None)
    _, kw = _mask_args(mask, window, segs)
    scale = D ** -0.5
    out, lse = ops.flash_fwd(q, k, v, softmax_scale=scale, **kw)
    dq, dk, dv = ops.flash_bwd(q, k, v, out, lse, do, softmax_scale=scale, ds_workspace=ds_workspace, **kw)
    torch.cuda.synchronize()
    G = Hq // Hkv
    w = window if mask == "sliding" else None
    for (b, hk) in samples:
        hs = slice(hk * G, (hk + 1) * G)
        for (k0, k1) in key_blocks:
            # dK/dV of keys [k0, k1): contributions come from query rows [k0, r_hi) only, and those rows
            # normalise over keys [s_lo, r_hi).
            r_hi = T if w is None else min(T, k1 + w)
            s_lo = 0 if w is None else max(0, k0 - w)
            qs, dos = q[b:b + 1, k0:r_hi, hs].cpu(), do[b:b + 1, k0:r_hi, hs].cpu()
            ks, vs = k[b:b + 1, s_lo:r_hi, hk:hk + 1].cpu(), v[b:b + 1, s_lo:r_hi, hk:hk + 1].cpu()
            sub = ref.MaskSpec(**spec_kw, target_positions=torch.arange(k0, r_hi)[None],
                               source_positions=torch.arange(s_lo, r_hi)[None])
            if segs is not None:
                keep = segs[b:b + 1, k0:r_hi, None] == segs[b:b + 1, None, s_lo:r_hi]
                sub.dense_bias = ref.bool_to_bias(keep)[:, None]
            _, wk, wv = ref.reference_mha_grads(qs, ks, vs, dos, sub, softmax_scale=scale, row_block=128)
            sl = slice(k0 - s_lo, k1 - s_lo)
            assert _rel_ok(dk[b:b + 1, k0:k1, hk:hk + 1].cpu(), wk[:, sl]), (
                "dk", b, hk, k0, ref.rel_l2(dk[b:b + 1, k0:k1, hk:hk + 1].cpu(), wk[:, sl]))
            assert _rel_ok(dv[b:b + 1, k0:k1, hk:hk + 1].cpu(), wv[:, sl]), (
                "dv", b, hk, k0, ref.rel_l2(dv[b:b + 1, k0:k1, hk:hk + 1].cpu(), wv[:, sl]))
        for (r0, r1) in dq_rows:
            # Query rows [r0, r1) against keys [0, r1): exact for causal / sliding masks.
            qs, ks, vs = q[b:b + 1, r0:r1, hs].cpu(), k[b:b + 1, :r1, hk:hk + 1].cpu(), v[b:b + 1, :r1, hk:hk + 1].cpu()
            sub = ref.MaskSpec(**spec_kw, segment_ids=None if segs is None else segs[b:b + 1, :r1],
                               target_positions=torch.arange(r0, r1)[None], source_positions=torch.arange(r1)[None])
            if segs is not None:
                # segment mask of the sub-problem: rows r0..r1 vs keys 0..r1
                sub.segment_ids = None
                keep = segs[b:b + 1, r0:r1, None] == segs[b:b + 1, None, :r1]
                sub.dense_bias = ref.bool_to_bias(keep)[:, None]
            want = ref.reference_mha(qs, ks, vs, sub, softmax_scale=scale, row_block=128)
            assert _rel_ok(out[b:b + 1, r0:r1, hs].cpu(), want), ("out", b, hk, r0)
            # dq of these rows only depends on these rows.
            wq, _, _ = ref.reference_mha_grads(qs, ks, vs, do[b:b + 1, r0:r1, hs].cpu(), sub, softmax_scale=scale, row_block=128)
            assert _rel_ok(dq[b:b + 1, r0:r1, hs].cpu(), wq), ("dq", b, hk, r0)
    # Identities over the whole tensors (fp32 sums of bf16 values).
    dv_sum = dv.float().sum(dim=1)                                   # [B, Hkv, D]
    do_sum = do.float().sum(dim=1).reshape(B, Hkv, G, D).sum(dim=2)
    assert ref.rel_l2(dv_sum.cpu(), do_sum.cpu()) < 1e-2
    dk_sum = dk.float().sum(dim=1)
    assert float(dk_sum.abs().max()) < 2e-2 * float(dk.float().abs().max()) * (T ** 0.5)
    return out, dq, dk, dv


@pytest.mark.parametrize("ds_workspace", [False, True])
def test_baseline_c2_full_size(ds_workspace):
    """C2 at full size (32 (batch, kv head) pairs: the per-XCD grouped block order), through the
    backward that recomputes dS for dq and through the one that keeps dS in the workspace.  Key blocks: the first, one
    in the middle and a late one that only 256 query rows see."""
    _sampled_fwd_bwd_check(4, 4096, 32, 8, 128, "causal", None, False,
                           samples=[(0, 0), (3, 7)], dq_rows=[(0, 128), (1920, 2048), (3968, 4096)],
                           key_blocks=[(0, 128), (2048, 2176), (3840, 3968)], ds_workspace=ds_workspace)


def test_baseline_c2_dkdv_sampled():
    """dK/dV of one (batch, kv head) at the C2 shape against the oracle on that whole group."""
    B, T, Hq, Hkv, D = 1, 4096, 4, 1, 128
    q, k, v, do = _inputs(B, T, Hq, Hkv, D, torch.bfloat16)
    scale = D ** -0.5
    spec = ref.MaskSpec(causal=True)
    wq, wk, wv = ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=scale, dtype=torch.float32)
    kw = dict(softmax_scale=scale, mask_kind=ops.MASK_CAUSAL)
    out, lse = ops.flash_fwd(q.cuda(), k.cuda(), v.cuda(), **kw)
    dq, dk, dv = ops.flash_bwd(q.cuda(), k.cuda(), v.cuda(), out, lse, do.cuda(), **kw)
    for name, got, want in (("dq", dq, wq), ("dk", dk, wk), ("dv", dv, wv)):
        _assert_close(name, got, want, torch.bfloat16)


def _doc_boundary(seed, batch, seq_len, b):
    """First position of row b's second document (or the middle of the row if it has one document)."""
    ids = ref.packed_segment_ids(seed, batch, seq_len)[b]
    change = torch.nonzero(ids[1:] != ids[:-1]).flatten()
    return int(change[0]) + 1 if len(change) else seq_len // 2


@pytest.mark.parametrize("ds_workspace", [False, True])
def test_baseline_c3_full_size(ds_workspace):
    """C3 at full size (128 pairs), through both backward paths.  Key blocks per sampled row: one that
    straddles a document boundary, one whose last visible query rows sit at the window edge
    (key + 4096 < T), a late one."""
    B, T = 8, 8192
    for b, hk in ((0, 0), (5, 11)):
        cut = _doc_boundary(4, B, T, b)
        straddle = (cut // 128) * 128 if cut % 128 else cut - 64  # 128 keys with the boundary inside
        straddle = max(0, min(T - 128, straddle))
        _sampled_fwd_bwd_check(B, T, 16, 16, 128, "sliding", 4096, True, samples=[(b, hk)],
                               dq_rows=[(0, 128), (4096, 4224), (8064, 8192)],
                               key_blocks=[(straddle, straddle + 128), (1024, 1152), (7936, 8064)],
                               ds_workspace=ds_workspace)


@pytest.mark.parametrize("ds_workspace", [False, True])
def test_baseline_c5_full_size(ds_workspace):
    _sampled_fwd_bwd_check(1, 32768, 64, 8, 128, "causal", None, False,
                           samples=[(0, 3)], dq_rows=[(0, 128), (16384, 16512), (32640, 32768)],
                           key_blocks=[(32384, 32512), (32000, 32128)], ds_workspace=ds_workspace)
