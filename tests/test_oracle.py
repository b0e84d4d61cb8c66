"""Pins the CPU oracle (oracle/) before anything is compared against it.

Checks are chosen so that a plausible mistake (dropped scale, wrong GQA grouping, off-by-one in the
window, transposed operand, wrong sign in dS) fails at least one of them.
"""

import json
import os

import numpy as np
import pytest
import scipy.special
import torch

from oracle import brute
from oracle import ref_attention as ref


def _rand(seed, shape):
    return np.random.default_rng(seed).standard_normal(shape)


# ------------------------------------------------------------------ masks: reference's own tables


def test_sliding_window_tables(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "mask_tables.json")))
    for case in g["sliding_window_5x5"]:
        fn = ref.sliding_window_causal_mask(case["left_context"])
        got = fn(np.arange(5)[:, None], np.arange(5)[None, :]).astype(np.int32)
        assert got.tolist() == case["expected"]
    for case in g["sliding_window2_with_time_step_3x5"]:
        fn = ref.sliding_window_causal_mask(2)
        got = fn(np.arange(3)[:, None] + case["time_step"], np.arange(5)[None, :]).astype(np.int32)
        assert got.tolist() == case["expected"]


def test_causal_and_segment_tables(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "mask_tables.json")))
    got = ref.causal_mask(np.arange(3)[:, None], np.arange(3)[None, :]).astype(np.int32)
    assert got.tolist() == g["causal_3x3"]
    bias = ref.bool_to_bias(ref.causal_mask(np.arange(3)[:, None], np.arange(3)[None, :]))
    assert bias[0, 1] == np.float32(-1e15) and bias[1, 0] == 0.0
    seg = g["segment_4x4"]
    got = ref.segment_mask(np.asarray(seg["target_segments"]), np.asarray(seg["source_segments"]))
    assert got[:, None].astype(np.int32).tolist() == seg["expected"]


def test_sliding_window_block_map_invariant(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "mask_tables.json")))["sliding_window_block_map_invariant"]
    for w in g["sliding_window_sz"]:
        for t in g["seq_len"]:
            for blk in g["block_size"]:
                kw = dict(q_seq_len=t, kv_seq_len=t, block_q=blk, block_k=blk)
                a = ref.build_mask(ref.sliding_window_causal_mask(w), **kw)
                b = ref.build_sliding_window_mask(**kw, sliding_window_size=w)
                assert (a == b).all(), (w, t, blk)


def test_mask_spec_sums_biases():
    seg = torch.tensor([[1, 1, 2, 2]], dtype=torch.int32)
    spec = ref.MaskSpec(causal=True, segment_ids=seg)
    bias = spec.bias_rows(1, 0, 4, 4, 4, torch.float32)[0, 0]
    assert bias[0, 0] == 0 and bias[3, 2] == 0
    assert bias[0, 1] == -1e15  # causal only
    assert bias[2, 0] == -1e15  # segment only
    assert bias[0, 3] == -2e15  # both: composite bias is a plain sum
    keep = spec.keep_rows(0, 4, 4, 4)[0]
    assert keep.int().tolist() == [[1, 0, 0, 0], [1, 1, 0, 0], [0, 0, 1, 0], [0, 0, 1, 1]]


# ------------------------------------------------------------------ forward values


@pytest.mark.parametrize("hq,hkv", [(4, 4), (4, 2), (4, 1)])
def test_forward_matches_scipy_softmax(hq, hkv):
    b, t, s, d = 2, 9, 13, 8
    q, k, v = _rand(1, (b, t, hq, d)), _rand(2, (b, s, hkv, d)), _rand(3, (b, s, hkv, d))
    scale = 0.37
    out, lse = ref.reference_mha(torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v),
                                 softmax_scale=scale, return_lse=True, row_block=4)
    g = hq // hkv
    kr, vr = np.repeat(k, g, axis=2), np.repeat(v, g, axis=2)  # common.py:475-484
    logits = np.einsum("bthd,bshd->bhts", q * scale, kr)
    p = scipy.special.softmax(logits, axis=-1)
    want = np.einsum("bhts,bshd->bthd", p, vr)
    np.testing.assert_allclose(out.numpy(), want, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(lse.numpy(), scipy.special.logsumexp(logits, axis=-1), rtol=1e-12, atol=1e-12)
    bo, bl = brute.attention_fwd(q, k, v, scale=scale)
    np.testing.assert_allclose(bo, want, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(bl, lse.numpy(), rtol=1e-12, atol=1e-12)


def test_forward_matches_torch_sdpa_causal():
    b, t, h, d = 2, 32, 3, 16
    q, k, v = (torch.from_numpy(_rand(i, (b, t, h, d))) for i in (4, 5, 6))
    scale = d ** -0.5
    got = ref.reference_mha(q, k, v, ref.MaskSpec(causal=True), softmax_scale=scale, row_block=8)
    want = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True, scale=scale
    ).transpose(1, 2)
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-12)
    bo, _ = brute.attention_fwd(q.numpy(), k.numpy(), v.numpy(), scale=scale, mask_kind=brute.MASK_CAUSAL)
    np.testing.assert_allclose(bo, want.numpy(), rtol=1e-12, atol=1e-12)


def test_closed_forms():
    b, t, h, d = 1, 16, 2, 8
    q, k = (torch.from_numpy(_rand(i, (b, t, h, d))) for i in (7, 8))
    v = torch.from_numpy(_rand(9, (b, t, h, d)))
    out = ref.reference_mha(q, k, v, ref.MaskSpec(causal=True))
    torch.testing.assert_close(out[:, 0], v[:, 0])  # causal row 0 sees only key 0
    const = torch.ones_like(v) * torch.arange(d, dtype=torch.float64)
    out = ref.reference_mha(q, k, const, ref.MaskSpec(causal=True))
    torch.testing.assert_close(out, const)  # uniform V => out == V
    # window 0 == attend to self only.
    out = ref.reference_mha(q, k, v, ref.MaskSpec(sliding_window=0))
    torch.testing.assert_close(out, v)
    # Fully masked row: the bias is additive and finite, and in fp32 (the reference's logits dtype
    # for fp32 inputs) x + -1e15 == -1e15, so the row becomes a uniform average over ALL keys.
    spec = ref.MaskSpec(dense_bias=torch.full((1, 1, t, t), ref.NEG_INF))
    out = ref.reference_mha(q.float(), k.float(), v.float(), spec, mode="faithful")
    torch.testing.assert_close(out, v.float().mean(dim=1, keepdim=True).expand_as(v), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("window", [None, 0, 3, 100])
@pytest.mark.parametrize("with_seg", [False, True])
def test_masks_against_brute_force(window, with_seg):
    b, t, hq, hkv, d = 2, 24, 4, 2, 8
    q, k, v = _rand(10, (b, t, hq, d)), _rand(11, (b, t, hkv, d)), _rand(12, (b, t, hkv, d))
    seg = ref.packed_segment_ids(3, b, t, max_docs=4) if with_seg else None
    spec = ref.MaskSpec(causal=window is None, sliding_window=window, segment_ids=seg)
    got, lse = ref.reference_mha(torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v), spec,
                                 softmax_scale=0.3, return_lse=True, row_block=5)
    kind = brute.MASK_CAUSAL if window is None else brute.MASK_SLIDING
    bo, bl = brute.attention_fwd(q, k, v, scale=0.3, mask_kind=kind, window=window or 0,
                                 segment_ids=None if seg is None else seg.numpy())
    np.testing.assert_allclose(got.numpy(), bo, rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(lse.numpy(), bl, rtol=1e-11, atol=1e-11)
    # Element-level check of the window edge via per-element python loop.
    keep = spec.keep_rows(0, t, t, t)
    for bi in range(b):
        for i in range(t):
            for j in range(t):
                want = i >= j and (window is None or i - j <= window)
                if seg is not None:
                    want = want and int(seg[bi, i]) == int(seg[bi, j])
                assert bool(keep[bi if keep.shape[0] > 1 else 0, i, j]) == want


def test_faithful_mode_close_to_highprec_bf16():
    b, t, hq, hkv, d = 1, 64, 4, 2, 32
    q = ref.normal_tensor(0, (b, t, hq, d), torch.bfloat16)
    k = ref.normal_tensor(1, (b, t, hkv, d), torch.bfloat16)
    v = ref.normal_tensor(2, (b, t, hkv, d), torch.bfloat16)
    spec = ref.MaskSpec(causal=True)
    hp = ref.reference_mha(q, k, v, spec, softmax_scale=d ** -0.5)
    fa = ref.reference_mha(q, k, v, spec, softmax_scale=d ** -0.5, mode="faithful")
    assert fa.dtype == torch.bfloat16
    assert ref.max_abs(fa, hp) < 2e-2


# ------------------------------------------------------------------ gradients


def _loss(q, k, v, do, scale, mask_kind, window, seg):
    out, _ = brute.attention_fwd(q, k, v, scale=scale, mask_kind=mask_kind, window=window, segment_ids=seg)
    return float((out * do).sum())


def test_gradients_finite_differences():
    b, t, hq, hkv, d = 1, 6, 4, 2, 3
    q, k, v, do = (_rand(i, s) for i, s in ((20, (b, t, hq, d)), (21, (b, t, hkv, d)), (22, (b, t, hkv, d)), (23, (b, t, hq, d))))
    seg = np.asarray([[1, 1, 1, 2, 2, 2]], dtype=np.int32)
    scale, kind, window = 0.7, brute.MASK_SLIDING, 2
    dq, dk, dv = brute.attention_bwd(q, k, v, do, scale=scale, mask_kind=kind, window=window, segment_ids=seg)
    eps = 1e-6
    for name, x, gx in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        num = np.zeros_like(x)
        it = np.nditer(x, flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            old = x[idx]
            x[idx] = old + eps
            fp = _loss(q, k, v, do, scale, kind, window, seg)
            x[idx] = old - eps
            fm = _loss(q, k, v, do, scale, kind, window, seg)
            x[idx] = old
            num[idx] = (fp - fm) / (2 * eps)
        np.testing.assert_allclose(gx, num, rtol=1e-6, atol=1e-7, err_msg=name)
    # Autodiff of the torch restatement agrees with the analytic brute force.
    spec = ref.MaskSpec(sliding_window=window, segment_ids=torch.from_numpy(seg))
    tq, tk, tv = ref.reference_mha_grads(*(torch.from_numpy(x) for x in (q, k, v, do)), spec,
                                         softmax_scale=scale, row_block=4)
    np.testing.assert_allclose(tq.numpy(), dq, rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(tk.numpy(), dk, rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(tv.numpy(), dv, rtol=1e-10, atol=1e-10)


def test_gradient_identities():
    b, t, h, d = 1, 12, 2, 4
    q, k, v, do = (_rand(i, (b, t, h, d)) for i in (30, 31, 32, 33))
    dq, dk, dv = brute.attention_bwd(q, k, v, do, scale=0.5, mask_kind=brute.MASK_CAUSAL)
    # Softmax is shift invariant: adding c*q-independent constant to all logits of a row changes
    # nothing, which makes sum_k dS_ik = 0; with K shifted by a common vector u the loss is constant
    # => sum over keys of dK equals 0 projected on any direction of q-space only if mask-free.
    dq0, dk0, dv0 = brute.attention_bwd(q, k, v, do, scale=0.5)
    np.testing.assert_allclose(dk0.sum(axis=1), 0.0, atol=1e-12)
    # dV column sums equal dO column sums (rows of P sum to 1).
    np.testing.assert_allclose(dv.sum(axis=1), do.sum(axis=1), atol=1e-12)
    np.testing.assert_allclose(dv0.sum(axis=1), do.sum(axis=1), atol=1e-12)
    assert np.abs(dq - dq0).max() > 1e-3


# ------------------------------------------------------------------ logit sink


def _sink_as_extra_key(q, k, v, sink, scale):
    """The sink written as an ordinary key, so that the sink-free oracle (pinned above) applies:
    one more coordinate holds sink_h / scale in the queries of head h, 1 in the extra key and 0 in
    the real keys, and the extra key's value row is zero."""
    b, t, hq, d = q.shape
    s, hkv = k.shape[1], k.shape[2]
    qa = np.concatenate([q, np.broadcast_to((sink / scale)[None, None, :, None], (b, t, hq, 1))], axis=-1)
    ka = np.zeros((b, s + 1, hkv, d + 1))
    ka[:, 1:, :, :d] = k
    ka[:, 0, :, d] = 1.0
    va = np.zeros((b, s + 1, hkv, d + 1))
    va[:, 1:, :, :d] = v
    return qa, ka, va


def test_logit_sink_equals_an_extra_key_with_zero_value():
    b, t, s, hq, hkv, d = 2, 7, 11, 4, 2, 5
    q, k, v, do = (_rand(i, sh) for i, sh in ((60, (b, t, hq, d)), (61, (b, s, hkv, d)), (62, (b, s, hkv, d)), (63, (b, t, hq, d))))
    sink = np.asarray([0.9, -1.3, 0.0, 2.5])
    scale = 0.41
    tq, tk, tv, tdo, tsink = (torch.from_numpy(x) for x in (q, k, v, do, sink))
    out, lse = ref.reference_mha(tq, tk, tv, softmax_scale=scale, logit_sink=tsink, return_lse=True, row_block=3)
    qa, ka, va = _sink_as_extra_key(q, k, v, sink, scale)
    want, want_lse = ref.reference_mha(*(torch.from_numpy(x) for x in (qa, ka, va)), softmax_scale=scale, return_lse=True)
    np.testing.assert_allclose(out.numpy(), want.numpy()[..., :d], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(lse.numpy(), want_lse.numpy(), rtol=1e-12, atol=1e-12)
    # The C brute force agrees on the augmented problem too.
    bo, _ = brute.attention_fwd(qa, ka, va, scale=scale)
    np.testing.assert_allclose(out.numpy(), bo[..., :d], rtol=1e-12, atol=1e-12)
    # Gradients: those of the real coordinates carry over; d sink_h = sum_{b,t} dq'[b,t,h,D] / scale.
    dq, dk, dv, dsink = ref.reference_mha_grads(tq, tk, tv, tdo, softmax_scale=scale, logit_sink=tsink, row_block=3)
    doa = np.concatenate([do, np.zeros((b, t, hq, 1))], axis=-1)
    aq, ak, av = brute.attention_bwd(qa, ka, va, doa, scale=scale)
    np.testing.assert_allclose(dq.numpy(), aq[..., :d], rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dk.numpy(), ak[:, 1:, :, :d], rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dv.numpy(), av[:, 1:, :, :d], rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dsink.numpy(), aq[..., d].sum(axis=(0, 1)) / scale, rtol=1e-10, atol=1e-12)


def test_logit_sink_closed_forms():
    b, t, h, d = 1, 8, 2, 4
    q, k, v = (torch.from_numpy(_rand(i, (b, t, h, d))) for i in (64, 65, 66))
    # Equal logits everywhere (q == 0) and sink 0: S + 1 equal weights, one of them on nothing.
    out = ref.reference_mha(torch.zeros_like(q), k, v, logit_sink=torch.zeros(h, dtype=torch.float64))
    torch.testing.assert_close(out, (v.sum(dim=1, keepdim=True) / (t + 1)).expand_as(v))
    # A sink far below every logit changes nothing; one far above takes all the mass.
    base = ref.reference_mha(q, k, v, ref.MaskSpec(causal=True))
    low = ref.reference_mha(q, k, v, ref.MaskSpec(causal=True), logit_sink=torch.full((h,), -1e4, dtype=torch.float64))
    torch.testing.assert_close(low, base)
    high = ref.reference_mha(q, k, v, ref.MaskSpec(causal=True), logit_sink=torch.full((h,), 1e4, dtype=torch.float64))
    assert high.abs().max() == 0
    # Causal row 0 sees key 0 and the sink: weight sigmoid(s00 - sink) on v0.  The mask bias does
    # not touch the sink (attention.py:596-598).
    sink = torch.tensor([0.3, -0.7], dtype=torch.float64)
    out, lse = ref.reference_mha(q, k, v, ref.MaskSpec(causal=True), logit_sink=sink, return_lse=True)
    s00 = (q[:, 0] * k[:, 0]).sum(-1)  # [b, h]
    torch.testing.assert_close(out[:, 0], torch.sigmoid(s00 - sink)[..., None] * v[:, 0])
    torch.testing.assert_close(lse[:, :, 0], torch.logaddexp(s00, sink.expand_as(s00)))


# ------------------------------------------------------------------ dense bias, dropout


def test_dense_bias_against_structured_masks_and_rank_one_form():
    b, t, hq, hkv, d = 2, 10, 4, 2, 6
    q, k, v = (torch.from_numpy(_rand(i, sh)) for i, sh in ((70, (b, t, hq, d)), (71, (b, t, hkv, d)), (72, (b, t, hkv, d))))
    seg = torch.tensor([[1, 1, 1, 2, 2, 2, 2, 3, 3, 3], [5, 5, 5, 5, 5, 0, 0, 0, 0, 0]], dtype=torch.int32)
    # The causal + segment mask written out as a dense bias of 0 / -1e15 entries.
    keep = (torch.arange(t)[:, None] >= torch.arange(t)[None, :])[None] & (seg[:, :, None] == seg[:, None, :])
    dense = torch.where(keep, 0.0, ref.NEG_INF)[:, None]
    want = ref.reference_mha(q, k, v, ref.MaskSpec(causal=True, segment_ids=seg), softmax_scale=0.3)
    got = ref.reference_mha(q, k, v, ref.MaskSpec(dense_bias=dense), softmax_scale=0.3)
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-12)
    # A rank-one bias u[b,h,t] + w[b,h,s] is the product of two augmented coordinates:
    # q' = [q, u/scale, 1/scale], k' = [k, 1, w]; needs one kv head per query head.
    hq = hkv
    q = q[:, :, :hkv]
    # Dyadic values: the oracle carries biases in fp32 (attention.py:579), where these sums are exact.
    u, w = np.round(_rand(73, (b, hq, t)) * 8) / 8, np.round(_rand(74, (b, hq, t)) * 8) / 8
    bias = torch.from_numpy(u[:, :, :, None] + w[:, :, None, :])
    scale = 0.3
    got, lse = ref.reference_mha(q, k, v, ref.MaskSpec(dense_bias=bias), softmax_scale=scale, return_lse=True)
    qa = np.concatenate([q.numpy(), u.transpose(0, 2, 1)[..., None] / scale, np.full((b, t, hq, 1), 1 / scale)], axis=-1)
    ka = np.concatenate([k.numpy(), np.ones((b, t, hkv, 1)), w.transpose(0, 2, 1)[..., None]], axis=-1)
    va = np.concatenate([v.numpy(), np.zeros((b, t, hkv, 2))], axis=-1)
    bo, bl = brute.attention_fwd(qa, ka, va, scale=scale)
    np.testing.assert_allclose(got.numpy(), bo[..., :d], rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(lse.numpy(), bl, rtol=1e-11, atol=1e-12)


def test_dropout_is_linear_in_the_value_rows():
    b, t, s, hq, hkv, d = 1, 5, 7, 4, 2, 3
    q, k, v = (torch.from_numpy(_rand(i, sh)) for i, sh in ((75, (b, t, hq, d)), (76, (b, s, hkv, d)), (77, (b, s, hkv, d))))
    rate = 0.3
    mask = torch.from_numpy(np.random.default_rng(78).random((b, hq, t, s)) < rate)
    assert mask.any() and not mask.all()
    got, lse = ref.reference_mha(q, k, v, softmax_scale=0.8, dropout_mask=mask, dropout_rate=rate, return_lse=True, row_block=2)
    base, base_lse = ref.reference_mha(q, k, v, softmax_scale=0.8, return_lse=True)
    torch.testing.assert_close(lse, base_lse)  # dropout acts after the softmax
    want = torch.zeros_like(got)
    for j in range(s):
        vj = torch.zeros_like(v)
        vj[:, j] = v[:, j]
        oj = ref.reference_mha(q, k, vj, softmax_scale=0.8)  # P[., j] * v_j, undropped (pinned above)
        keep = (~mask[:, :, :, j]).permute(0, 2, 1)[..., None].to(oj.dtype)  # [b, t, hq, 1]
        want += keep * oj / (1 - rate)
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-12)
    # Nothing dropped: a pure rescale.
    none = ref.reference_mha(q, k, v, softmax_scale=0.8, dropout_mask=torch.zeros_like(mask), dropout_rate=rate)
    torch.testing.assert_close(none, base / (1 - rate))


def test_dropout_bias_sink_gradients_finite_differences():
    b, t, hq, hkv, d = 1, 5, 2, 1, 3
    rng = np.random.default_rng(79)
    q, k, v, do = (rng.standard_normal(sh) for sh in ((b, t, hq, d), (b, t, hkv, d), (b, t, hkv, d), (b, t, hq, d)))
    sink = rng.standard_normal(hq)
    bias = torch.from_numpy(rng.standard_normal((1, hq, t, t)))
    rate = 0.25
    mask = torch.from_numpy(rng.random((b, hq, t, t)) < rate)
    spec = ref.MaskSpec(causal=True, dense_bias=bias)
    kw = dict(softmax_scale=0.6, dropout_mask=mask, dropout_rate=rate)

    def loss(q_, k_, v_, s_):
        out = ref.reference_mha(*(torch.from_numpy(x) for x in (q_, k_, v_)), spec, logit_sink=torch.from_numpy(s_), **kw)
        return float((out * torch.from_numpy(do)).sum())

    grads = ref.reference_mha_grads(*(torch.from_numpy(x) for x in (q, k, v, do)), spec,
                                    logit_sink=torch.from_numpy(sink), row_block=2, **kw)
    eps = 1e-6
    args = [q, k, v, sink]
    for i, name in enumerate(("q", "k", "v", "sink")):
        x = args[i]
        num = np.zeros_like(x)
        it = np.nditer(x, flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            old = x[idx]
            x[idx] = old + eps
            fp = loss(*args)
            x[idx] = old - eps
            fm = loss(*args)
            x[idx] = old
            num[idx] = (fp - fm) / (2 * eps)
        np.testing.assert_allclose(grads[i].numpy(), num, rtol=1e-6, atol=1e-7, err_msg=name)


# ------------------------------------------------------------------ paged KV / decode


def test_reconstruct_kv_loop():
    hkv, total, page, d, b, pps = 2, 6, 4, 3, 2, 3
    pages = torch.arange(hkv * total * page * d, dtype=torch.float32).reshape(hkv, total, page, d)
    tables = torch.tensor([[5, 0, 2], [1, 7, 3]], dtype=torch.int32)  # 7 is out of range -> zeros
    got = ref.reconstruct_kv(tables, pages)
    assert got.shape == (b, pps * page, hkv, d)
    for bi in range(b):
        for j in range(pps * page):
            pg = int(tables[bi, j // page])
            for h in range(hkv):
                want = pages[h, pg, j % page] if pg < total else torch.zeros(d)
                assert torch.equal(got[bi, j, h], want)


def test_reconstruct_kv_negative_and_out_of_pool_indices_loop():
    """`pages.at[:, page_tables].get(mode="fill", fill_value=0)` (kv_cache/paged_kv_cache.py:32) is
    jax.numpy indexing (jax 0.8.3, pyproject.toml:25; not under the reference tree): a signed index
    is first normalised the numpy way, i + size if i < 0, and only what is still outside [0, size)
    afterwards is out of bounds and reads the fill value.  Spelled out element by element."""
    hkv, total, page, d, pps = 2, 5, 2, 3, 7
    pages = torch.arange(1, 1 + hkv * total * page * d, dtype=torch.float32).reshape(hkv, total, page, d)
    tables = torch.tensor([[-1, -5, -6, 4, 5, 0, -2], [2, -total, total, -total - 1, 1, -3, 3]], dtype=torch.int32)
    got = ref.reconstruct_kv(tables, pages)
    assert got.shape == (2, pps * page, hkv, d)
    for bi in range(2):
        for j in range(pps * page):
            idx = int(tables[bi, j // page])
            if idx < 0:
                idx += total            # -1 is the last page, -total the first
            for h in range(hkv):
                if 0 <= idx < total:
                    assert torch.equal(got[bi, j, h], pages[h, idx, j % page]), (bi, j, h)
                else:                   # below -total or at / above total: the fill value
                    assert torch.equal(got[bi, j, h], torch.zeros(d)), (bi, j, h)
    # the entries above cover: wrap to the last / first page, one past either end, and plain indices
    assert int((got == 0).all(dim=-1).sum()) == 4 * page * hkv


def _bf16_round(x: float) -> float:
    """Round-to-nearest-even of a double to bfloat16, by bit manipulation of its float32 pattern
    (independent of torch's conversion)."""
    import struct

    bits = struct.unpack("<I", struct.pack("<f", x))[0]
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return struct.unpack("<f", struct.pack("<I", bits))[0]


def test_faithful_mode_rounding_points_by_hand():
    """The "faithful" mode keeps ReferenceMHA's rounding points for bf16 inputs (q * scale in bf16,
    flash_attention/common.py:505; logits in bf16, :510; fp32 softmax rounded back to bf16,
    attention.py:604-625; context in bf16, common.py:519).  Two keys, head_dim 1, numbers chosen so
    that every rounding point moves the result by more than a bf16 step: worked with python floats."""
    import math

    scale, q, k0, k1, v0, v1 = 0.3, 1.0, 100.0, 99.0, 1.0, 0.0
    qs = _bf16_round(q * scale)                                         # 0.30078125
    assert qs == 0.30078125
    l0, l1 = _bf16_round(qs * k0), _bf16_round(qs * k1)                # 30.125, 29.75
    assert (l0, l1) == (30.125, 29.75)
    p0 = 1.0 / (1.0 + math.exp(l1 - l0))
    p0r, p1r = _bf16_round(p0), _bf16_round(1.0 - p0)
    want = _bf16_round(p0r * v0 + p1r * v1)                             # 0.59375
    assert want == 0.59375
    # what the result would be with the rounding of q * scale left out, for contrast
    no_q_round = _bf16_round(_bf16_round(1.0 / (1.0 + math.exp(_bf16_round(0.3 * k1) - _bf16_round(0.3 * k0)))))
    assert no_q_round == 0.5625 and no_q_round != want
    qt = torch.tensor([[[[q]]]], dtype=torch.bfloat16)                 # [B=1, T=1, H=1, D=1]
    kt = torch.tensor([[[[k0]], [[k1]]]], dtype=torch.bfloat16)        # [1, S=2, 1, 1]
    vt = torch.tensor([[[[v0]], [[v1]]]], dtype=torch.bfloat16)
    got = ref.reference_mha(qt, kt, vt, ref.MaskSpec(), softmax_scale=scale, mode="faithful")
    assert got.dtype == torch.bfloat16 and float(got[0, 0, 0, 0]) == want
    # the high-precision mode rounds nowhere: sigmoid(0.3) exactly
    hp = ref.reference_mha(qt, kt, vt, ref.MaskSpec(), softmax_scale=scale)
    assert abs(float(hp[0, 0, 0, 0]) - 1.0 / (1.0 + math.exp(-0.3))) < 1e-12


def test_scatter_update_pages_loop():
    """The oracle's page insert against the element-wise loop documented in
    kv_cache/paged_kv_cache.py:156-165, with the GPU kernel's guards (paged_kv_cache_gpu_kernel.py:26,31):
    position out of range -> nothing; page 0 -> nothing; page outside the pool -> dropped."""
    h, total, page, d, b, pps = 2, 7, 4, 3, 5, 3
    pages = torch.arange(h * total * page * d, dtype=torch.float32).reshape(h, total, page, d)
    proj = -1.0 - torch.arange(h * b * d, dtype=torch.float32).reshape(h, b, 1, d)
    tables = torch.tensor([[5, 1, 2], [3, 0, 4], [6, 6, 6], [2, 9, 1], [4, 3, 5]], dtype=torch.int32)
    pos = torch.tensor([[6], [5], [12], [4], [-1]], dtype=torch.int32)
    # seq 0 -> page 1 row 2; seq 1 -> page 0 (padding, skipped); seq 2 -> pos 12 out of range;
    # seq 3 -> page 9 outside the pool (dropped); seq 4 -> negative position.
    got = ref.scatter_update_pages(pages, proj, tables, pos)
    want = pages.clone()
    for i in range(b):
        p = int(pos[i, 0])
        if p < 0 or p >= page * pps:
            continue
        actual = int(tables[i, p // page])
        if actual == 0 or actual >= total:
            continue
        for kh in range(h):
            for e in range(d):
                want[kh, actual, p % page, e] = proj[kh, i, 0, e]
    assert torch.equal(got, want)
    assert int((got != pages).any(dim=-1).sum()) == h  # exactly one row per head changed
    # Round trip: the inserted token shows up at its position in the gathered cache.
    dense = ref.reconstruct_kv(tables, got)
    assert torch.equal(dense[0, 6], proj[:, 0, 0])
    # One position broadcast over the batch (paged_kv_cache.py:216-217).
    tables2 = torch.tensor([[1, 2], [3, 4]], dtype=torch.int32)
    got2 = ref.scatter_update_pages(pages, proj[:, :2], tables2, torch.tensor([[5]], dtype=torch.int32))
    assert torch.equal(got2[:, 2, 1], proj[:, 0, 0]) and torch.equal(got2[:, 4, 1], proj[:, 1, 0])


def test_paged_decode_equals_dense_and_brute():
    b, hq, hkv, d, page, pps = 3, 4, 2, 8, 4, 5
    q, k, v, tables, lengths = ref.paged_inputs(7, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                page_size=page, pages_per_seq=pps, min_len=1,
                                                max_len=page * pps, dtype=torch.float64)
    got = ref.reference_decode(q, k, v, lengths, softmax_scale=0.4, page_tables=tables)
    dense_k, dense_v = ref.reconstruct_kv(tables, k), ref.reconstruct_kv(tables, v)
    want = ref.reference_decode(q, dense_k, dense_v, lengths, softmax_scale=0.4)
    torch.testing.assert_close(got, want, rtol=0, atol=0)
    bo = brute.paged_decode(q[:, 0].numpy(), k.numpy(), v.numpy(), tables.numpy(), lengths.numpy(), scale=0.4)
    np.testing.assert_allclose(got[:, 0].numpy(), bo, rtol=1e-12, atol=1e-12)
    # Decode == last valid row of a causal prefill over the same keys.
    for bi in range(b):
        n = int(lengths[bi])
        qq = torch.zeros((1, n, hq, d), dtype=torch.float64)
        qq[0, n - 1] = q[bi, 0]
        full = ref.reference_mha(qq, dense_k[bi : bi + 1, :n], dense_v[bi : bi + 1, :n],
                                 ref.MaskSpec(causal=True), softmax_scale=0.4)
        torch.testing.assert_close(full[0, n - 1], got[bi, 0], rtol=1e-12, atol=1e-12)
    # Sliding window in decode.
    gw = ref.reference_decode(q, k, v, lengths, softmax_scale=0.4, page_tables=tables, sliding_window=3)
    bw = brute.paged_decode(q[:, 0].numpy(), k.numpy(), v.numpy(), tables.numpy(), lengths.numpy(), scale=0.4, window=3)
    np.testing.assert_allclose(gw[:, 0].numpy(), bw, rtol=1e-12, atol=1e-12)


def test_page_permutation_invariance():
    b, hq, hkv, d, page, pps = 2, 2, 1, 4, 2, 4
    q, k, v, tables, lengths = ref.paged_inputs(9, batch=b, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                                page_size=page, pages_per_seq=pps, min_len=2,
                                                max_len=page * pps, dtype=torch.float64)
    base = ref.reference_decode(q, k, v, lengths, page_tables=tables)
    perm = torch.from_numpy(np.random.default_rng(0).permutation(b * pps))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(b * pps)
    k2, v2 = k[:, perm], v[:, perm]
    tables2 = inv[tables.long()].to(torch.int32)
    again = ref.reference_decode(q, k2, v2, lengths, page_tables=tables2)
    assert torch.equal(base, again)


def test_synthetic_generators():
    seg = ref.packed_segment_ids(4, 8, 8192)
    assert seg.shape == (8, 8192) and seg.dtype == torch.int32
    assert int(seg.min()) == 1 and int(seg.max()) <= 6
    assert bool((seg[:, 1:] >= seg[:, :-1]).all())
    spec = ref.MaskSpec(causal=True)
    assert ref.count_unmasked_pairs(spec, 2, 64, 64, row_block=16) == 2 * 64 * 65 // 2
    a = ref.normal_tensor(0, (4, 4), torch.bfloat16)
    b = ref.normal_tensor(0, (4, 4), torch.bfloat16)
    assert torch.equal(a, b)
