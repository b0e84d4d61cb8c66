"""CPU restatement of AXLearn's XLA reference attention. TEST INFRASTRUCTURE ONLY.

This module is the checker the HIP kernels are compared against. It is never imported by the
product package `axlearn_amd`; only tests, the smoke check and the CPU-baseline leg of the benchmark
may use it.

Reference files restated here (paths relative to the apple/axlearn checkout):

* `axlearn/common/flash_attention/common.py:492-519` (`ReferenceMHA.__call__`): scale the query
  first, gather pages if paged, GQA logits, softmax with the summed biases, GQA context.
* `axlearn/common/attention.py:565-631` (`apply_attention_logit_biases`, `softmax_with_biases`):
  bias is cast to the logits dtype before the add; 16-bit logits are up-cast to fp32 for the
  softmax; probabilities are cast back to the logits dtype.
* `axlearn/common/attention.py:2329-2380` (`compute_gqa_logits`, `compute_gqa_context`): query head
  `n` reads kv head `n // (Hq / Hkv)`.
* `axlearn/common/attention_bias.py:43` (`NEG_INF = -1e15`), `:243-246` (composite bias = plain sum
  of member biases), `:652-658` (`causal_mask`), `:771-790` (`sliding_window_causal_mask`),
  `:862-873` (`bool_to_bias`), `:876-882` (`_make_bool_segment_mask`).
* `axlearn/common/kv_cache/paged_kv_cache.py:21-34` (`reconstruct_kv`): page gather, out-of-range
  page index reads as zeros.
* `axlearn/common/kv_cache/paged_kv_cache_gpu_kernel.py:16-33` (`_scatter_pages_kernel`): insertion
  of the new token into the pool.
* `axlearn/common/flash_attention/gpu_decoding.py:314`, `gpu_paged_attention.py:344`:
  decode length = `target_positions[:, -1] + 1`.

Parity status of each function (what pins it, see tests/test_oracle.py):

* mask functions: pinned by the literal tables held in the reference's own tests
  (`attention_bias_test.py:27-53`, `attention_test.py:195-217`), committed under tests/golden.
* `reference_mha` values: the reference holds NO golden output vectors for attention values (all its
  tests are differential), so absolute values are pinned by mathematics instead: scipy softmax /
  logsumexp, torch's scaled_dot_product_attention, the C brute force in oracle/brute_force.c,
  closed-form special cases (uniform V, causal row 0, GQA == MHA on repeated KV).
* gradients: pinned by float64 central finite differences and by the independent analytic
  brute force in oracle/brute_force.c.
* logit sink: pinned by rewriting the sink as one more key with a zero value row (an extra head-dim
  coordinate carries sink / scale), which the sink-free functions and the C brute force evaluate,
  gradients included; plus closed forms (equal logits, sigmoid for a single visible key).
* dropout with a given mask: pinned by linearity in V (the output for mask M is the sum over keys j
  of (1 - M[., j]) / (1 - rate) times the output for V with only row j kept) and by float64 finite
  differences for the gradients.  The reference draws its masks with JAX's PRNG, which is not
  reproduced here: parity is defined for a given mask.
* dense bias: a bias that repeats the causal / segment mask as -1e15 entries must equal the
  structured mask; a rank-one bias u_t + w_s is absorbed into augmented q / k coordinates.
* `reconstruct_kv`: pinned by a pure-Python loop on tiny shapes.
* `scatter_update_pages`: pinned by the element-wise loop the reference documents
  (paged_kv_cache.py:156-165) written out in pure Python, plus the round trip through
  `reconstruct_kv`; the padding-page and out-of-range rules are read from the kernel source.
* XLA:CPU's exact bf16 rounding order inside einsum/softmax cannot be reproduced bit-for-bit without
  running jaxlib (absent here): "faithful" mode reproduces the rounding POINTS only.  parity unpinned
  at ULP level for the bf16 faithful mode; covered by the bf16 tolerance.
"""

from __future__ import annotations

import dataclasses
import math
from typing import Optional

import numpy as np
import torch

NEG_INF = -1e15  # attention_bias.py:43


# ----------------------------------------------------------------------------------------------
# Mask algebra (bit-exact integer / boolean work).
# ----------------------------------------------------------------------------------------------


def causal_mask(query_position, key_position):
    """attention_bias.py:652-658."""
    return query_position >= key_position


def sliding_window_causal_mask(sliding_window_size: int):
    """attention_bias.py:771-790. Keeps `sliding_window_size + 1` keys (self + window to the left)."""
    if sliding_window_size < 0:
        raise ValueError(f"{sliding_window_size=} must be a natural number.")

    def mask(query_position, key_position):
        return (query_position >= key_position) & (
            query_position - key_position <= sliding_window_size
        )

    return mask


def segment_mask(target_segments, source_segments):
    """attention_bias.py:876-882: [..., T] x [..., S] -> [..., T, S] equality (id 0 included)."""
    return target_segments[..., :, None] == source_segments[..., None, :]


def bool_to_bias(mask):
    """attention_bias.py:862-873: True -> 0, False -> NEG_INF."""
    if mask.dtype not in (torch.bool, np.bool_):
        raise ValueError("mask must be a Boolean tensor.")
    if isinstance(mask, np.ndarray):
        return (~mask).astype(np.float32) * np.float32(NEG_INF)
    return (~mask).to(torch.float32) * NEG_INF


@dataclasses.dataclass
class MaskSpec:
    """Structured description of the composite bias the BASELINE configs use.

    The composite bias is the SUM of the member biases (attention_bias.py:243-246), so an element
    masked by both the positional mask and the segment mask gets -2e15.
    """

    causal: bool = False
    sliding_window: Optional[int] = None  # implies causal; keeps window+1 keys
    segment_ids: Optional[torch.Tensor] = None  # [B, T] int32, T == S
    target_positions: Optional[torch.Tensor] = None  # [1|B, T] int
    source_positions: Optional[torch.Tensor] = None  # [1|B, S] int
    dense_bias: Optional[torch.Tensor] = None  # [1|B, 1|H, T, S] float

    def bias_rows(self, batch: int, t0: int, t1: int, q_len: int, kv_len: int, dtype) -> Optional[torch.Tensor]:
        """Returns the summed bias for query rows [t0, t1): shape [1|B, 1|H, t1-t0, S], or None."""
        total = None

        def add(x):
            nonlocal total
            total = x if total is None else total + x

        if self.causal or self.sliding_window is not None:
            tp = self.target_positions
            sp = self.source_positions
            if tp is None:
                tp = torch.arange(q_len, dtype=torch.int64)[None]
            if sp is None:
                sp = torch.arange(kv_len, dtype=torch.int64)[None]
            qp = tp[:, t0:t1, None].to(torch.int64)
            kp = sp[:, None, :].to(torch.int64)
            if self.sliding_window is not None:
                keep = sliding_window_causal_mask(self.sliding_window)(qp, kp)
            else:
                keep = causal_mask(qp, kp)
            add(bool_to_bias(keep)[:, None])
        if self.segment_ids is not None:
            seg = self.segment_ids
            keep = segment_mask(seg[:, t0:t1], seg)
            add(bool_to_bias(keep)[:, None])
        if self.dense_bias is not None:
            add(self.dense_bias[:, :, t0:t1, :].to(torch.float32))
        if total is None:
            return None
        return total.to(dtype)

    def keep_rows(self, t0: int, t1: int, q_len: int, kv_len: int) -> Optional[torch.Tensor]:
        """Boolean keep-mask for rows [t0,t1): [1|B, t1-t0, S] (dense bias ignored), or None."""
        keep = None
        if self.causal or self.sliding_window is not None:
            tp = self.target_positions
            sp = self.source_positions
            if tp is None:
                tp = torch.arange(q_len, dtype=torch.int64)[None]
            if sp is None:
                sp = torch.arange(kv_len, dtype=torch.int64)[None]
            qp = tp[:, t0:t1, None].to(torch.int64)
            kp = sp[:, None, :].to(torch.int64)
            if self.sliding_window is not None:
                keep = sliding_window_causal_mask(self.sliding_window)(qp, kp)
            else:
                keep = causal_mask(qp, kp)
        if self.segment_ids is not None:
            s = segment_mask(self.segment_ids[:, t0:t1], self.segment_ids)
            keep = s if keep is None else keep & s
        return keep


# ----------------------------------------------------------------------------------------------
# Paged KV.
# ----------------------------------------------------------------------------------------------


def reconstruct_kv(page_tables: torch.Tensor, pages: torch.Tensor) -> torch.Tensor:
    """kv_cache/paged_kv_cache.py:21-34.

    page_tables [B, pages_per_seq] int; pages [Hkv, P, page_size, D]
    -> [B, pages_per_seq * page_size, Hkv, D]; out-of-range indices read as zeros.
    """
    n, total, page_size, d = pages.shape
    b, pps = page_tables.shape
    idx = page_tables.to(torch.int64)
    # jnp `.at[].get(mode="fill")` wraps negative indices python-style before the range check.
    idx = torch.where(idx < 0, idx + total, idx)
    oob = (idx < 0) | (idx >= total)
    safe = idx.clamp(0, total - 1)
    g = pages[:, safe]  # [n, b, pps, page_size, d]
    g = torch.where(oob[None, :, :, None, None], torch.zeros((), dtype=pages.dtype), g)
    return g.permute(1, 2, 3, 0, 4).reshape(b, pps * page_size, n, d)


def scatter_update_pages(kv_pages: torch.Tensor, kv_proj: torch.Tensor, page_indices: torch.Tensor,
                         key_positions: torch.Tensor) -> torch.Tensor:
    """Insertion of one new token per sequence into a paged pool, as the reference's GPU kernel does it
    (kv_cache/paged_kv_cache_gpu_kernel.py:16-33; the loop it stands for is spelled out in
    kv_cache/paged_kv_cache.py:156-165).

    kv_pages [H, P, page_size, D]; kv_proj [H, B, 1, D]; page_indices [B, pps]; key_positions [B, 1].
    Returns an updated copy.  A position outside [0, page_size * pps) writes nothing (:26), page 0 (the
    padding page) is never written (:31), a page index outside the pool is dropped
    (paged_kv_cache.py:56-58, mode="drop").  A negative page index is undefined in the reference kernel;
    it is dropped here (parity unpinned for that case)."""
    out = kv_pages.clone()
    h, total, page_size, _ = kv_pages.shape
    b, pps = page_indices.shape
    for bi in range(b):
        pos = int(key_positions[bi if key_positions.shape[0] > 1 else 0, 0])
        if not 0 <= pos < page_size * pps:
            continue
        page = int(page_indices[bi, pos // page_size])
        if page <= 0 or page >= total:
            continue
        out[:, page, pos % page_size] = kv_proj[:, bi, 0].to(out.dtype)
    return out


# ----------------------------------------------------------------------------------------------
# ReferenceMHA restatement.
# ----------------------------------------------------------------------------------------------


def _round_to(x: torch.Tensor, dtype) -> torch.Tensor:
    return x.to(dtype)


def reference_mha(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    mask: Optional[MaskSpec] = None,
    *,
    softmax_scale: float = 1.0,
    mode: str = "highprec",
    page_tables: Optional[torch.Tensor] = None,
    row_block: int = 512,
    return_lse: bool = False,
    logit_sink: Optional[torch.Tensor] = None,
    dropout_mask: Optional[torch.Tensor] = None,
    dropout_rate: float = 0.0,
):
    """`ReferenceMHA.__call__` (flash_attention/common.py:492-519), query-row-blocked.

    dropout_mask [B,Hq,T,S] bool (True = dropped) with dropout_rate: `dropout(probs, rate, mask)`
    (flash_attention/common.py:512-518, layers.py:145-166) = where(mask, 0, probs) / (1 - rate),
    applied to the finished probabilities; lse is unaffected.

    logit_sink [Hq]: `softmax_with_biases` (attention.py:608-626) prepends it to every row of head
    h's biased logits, takes the softmax over S+1 entries and drops the sink's column again, so the
    returned probabilities sum to less than 1.  The returned lse includes the sink.

    query [B,T,Hq,D]; key/value [B,S,Hkv,D] (or page pools [Hkv,P,page,D] with `page_tables`).

    mode:
      "faithful": keeps the reference's rounding points for the input dtype: q*scale, logits,
          bias, probs and context are each rounded to the input dtype; softmax in fp32.
      "highprec": same operation order in float64 on the given (already rounded) inputs; output
          float64.  This is "fp32 accumulation" taken to its limit and is what kernels are held to.

    Returns context [B,T,Hq,D] (and lse [B,Hq,T] float64/fp32 of the biased, scaled logits).
    """
    mask = mask or MaskSpec()
    if page_tables is not None:
        key = reconstruct_kv(page_tables, key)
        value = reconstruct_kv(page_tables, value)
    b, t, hq, d = query.shape
    s, hkv = key.shape[1], key.shape[2]
    assert hq % hkv == 0
    g = hq // hkv
    in_dtype = query.dtype
    if mode == "highprec":
        cdt = torch.float64
        q = query.to(cdt) * softmax_scale
    elif mode == "faithful":
        cdt = torch.float32
        q = _round_to(query * softmax_scale, in_dtype).to(cdt)  # common.py:505 (in input dtype)
    else:
        raise ValueError(mode)
    k = key.to(cdt)
    v = value.to(cdt)
    out = torch.empty((b, t, hq, d), dtype=cdt)
    lse = torch.empty((b, hq, t), dtype=cdt)
    # [B, Hkv, S, D]
    kt = k.permute(0, 2, 1, 3)
    vt = v.permute(0, 2, 1, 3)
    for t0 in range(0, t, row_block):
        t1 = min(t, t0 + row_block)
        qb = q[:, t0:t1].reshape(b, t1 - t0, hkv, g, d).permute(0, 2, 3, 1, 4)  # b k g t d
        logits = torch.einsum("bkgtd,bksd->bkgts", qb, kt).reshape(b, hq, t1 - t0, s)
        if mode == "faithful":
            logits = _round_to(logits, in_dtype)
            bias = mask.bias_rows(b, t0, t1, t, s, in_dtype)  # attention.py:579
            if bias is not None:
                logits = _round_to(logits.to(torch.float32) + bias.to(torch.float32), in_dtype)
            logits = logits.to(torch.float32)
        else:
            bias = mask.bias_rows(b, t0, t1, t, s, torch.float32)
            if bias is not None:
                logits = logits + bias.to(cdt)
        if logit_sink is not None:
            sink = logit_sink.to(logits.dtype).reshape(1, hq, 1, 1).expand(b, hq, t1 - t0, 1)
            with_sink = torch.cat([sink, logits], dim=-1)
            m = with_sink.max(dim=-1, keepdim=True).values
            e_all = torch.exp(with_sink - m)
            z = e_all.sum(dim=-1, keepdim=True)
            probs = (e_all / z)[..., 1:]
        else:
            m = logits.max(dim=-1, keepdim=True).values
            e = torch.exp(logits - m)
            z = e.sum(dim=-1, keepdim=True)
            probs = e / z
        lse[:, :, t0:t1] = (m + torch.log(z)).squeeze(-1)
        if mode == "faithful":
            probs = _round_to(probs, in_dtype).to(cdt)
        if dropout_mask is not None:
            probs = torch.where(dropout_mask[:, :, t0:t1], torch.zeros_like(probs), probs) / (1.0 - dropout_rate)
            if mode == "faithful":
                probs = _round_to(probs, in_dtype).to(cdt)
        pb = probs.reshape(b, hkv, g, t1 - t0, s)
        ctx = torch.einsum("bkgts,bksd->btkgd", pb, vt).reshape(b, t1 - t0, hq, d)
        out[:, t0:t1] = ctx
    if mode == "faithful":
        out = _round_to(out, in_dtype)
    if return_lse:
        return out, lse
    return out


def reference_mha_grads(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    d_out: torch.Tensor,
    mask: Optional[MaskSpec] = None,
    *,
    softmax_scale: float = 1.0,
    row_block: int = 512,
    dtype=torch.float64,
    logit_sink: Optional[torch.Tensor] = None,
    dropout_mask: Optional[torch.Tensor] = None,
    dropout_rate: float = 0.0,
):
    """Gradients of `sum(reference_mha(q,k,v) * d_out)` w.r.t. q, k, v (and the logit sink, returned
    as a fourth tensor when one is given) by reverse-mode autodiff of the restatement above, in
    `dtype` on the given inputs, query-row-blocked.

    The reference obtains these from `jax.grad` of `ReferenceMHA` (gpu_attention_test.py:59-92).
    """
    mask = mask or MaskSpec()
    b, t, hq, d = query.shape
    s, hkv = key.shape[1], key.shape[2]
    g = hq // hkv
    k = key.to(dtype).clone().requires_grad_(True)
    v = value.to(dtype).clone().requires_grad_(True)
    dq = torch.empty((b, t, hq, d), dtype=dtype)
    do = d_out.to(dtype)
    sink = None if logit_sink is None else logit_sink.to(dtype).clone().requires_grad_(True)
    for t0 in range(0, t, row_block):
        t1 = min(t, t0 + row_block)
        qb_leaf = query[:, t0:t1].to(dtype).clone().requires_grad_(True)
        qb = (qb_leaf * softmax_scale).reshape(b, t1 - t0, hkv, g, d).permute(0, 2, 3, 1, 4)
        logits = torch.einsum("bkgtd,bksd->bkgts", qb, k.permute(0, 2, 1, 3)).reshape(b, hq, t1 - t0, s)
        bias = mask.bias_rows(b, t0, t1, t, s, torch.float32)
        if bias is not None:
            logits = logits + bias.to(dtype)
        if sink is not None:
            col = sink.reshape(1, hq, 1, 1).expand(b, hq, t1 - t0, 1)
            probs = torch.softmax(torch.cat([col, logits], dim=-1), dim=-1)[..., 1:]
        else:
            probs = torch.softmax(logits, dim=-1)
        if dropout_mask is not None:
            probs = torch.where(dropout_mask[:, :, t0:t1], torch.zeros_like(probs), probs) / (1.0 - dropout_rate)
        probs = probs.reshape(b, hkv, g, t1 - t0, s)
        ctx = torch.einsum("bkgts,bksd->btkgd", probs, v.permute(0, 2, 1, 3)).reshape(b, t1 - t0, hq, d)
        (ctx * do[:, t0:t1]).sum().backward()
        dq[:, t0:t1] = qb_leaf.grad
    if sink is not None:
        return dq, k.grad, v.grad, sink.grad
    return dq, k.grad, v.grad


def reference_decode(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    lengths: torch.Tensor,
    *,
    softmax_scale: float = 1.0,
    sliding_window: Optional[int] = None,
    page_tables: Optional[torch.Tensor] = None,
    mode: str = "highprec",
    dense_bias: Optional[torch.Tensor] = None,
):
    """Single-token decode through `ReferenceMHA` with a causal bias whose only query position is
    `lengths - 1` (decoding_test.py:131: `query_offset = seq_len - padding - 1`).

    query [B,1,Hq,D]; key/value [B,S,Hkv,D] or page pools + page_tables; lengths [B] int;
    dense_bias [1|B, 1|Hq, 1, S]: an explicit bias summed with the causal one, as the composite bias
    of a decode call sums its members (attention_bias.py:243-246; decoding_test.py:118-127 builds it).
    """
    b = query.shape[0]
    if page_tables is not None:
        kv_len = page_tables.shape[1] * key.shape[2]
    else:
        kv_len = key.shape[1]
    tp = (lengths.to(torch.int64) - 1).reshape(b, 1)
    spec = MaskSpec(
        causal=True,
        sliding_window=sliding_window,
        target_positions=tp,
        source_positions=torch.arange(kv_len, dtype=torch.int64)[None],
        dense_bias=dense_bias,
    )
    return reference_mha(
        query, key, value, spec, softmax_scale=softmax_scale, mode=mode, page_tables=page_tables
    )


# ----------------------------------------------------------------------------------------------
# Block maps (trace-time helpers of the reference), restated with plain numpy.
# ----------------------------------------------------------------------------------------------


def build_mask(mask_fn, *, q_seq_len: int, kv_seq_len: int, block_q: int, block_k: int) -> np.ndarray:
    """flash_attention/common.py:33-80: True where the (q-block, kv-block) tile keeps any element."""
    nq = -(-q_seq_len // block_q)
    nk = -(-kv_seq_len // block_k)
    out = np.ones((nq, nk), dtype=np.bool_)
    for i in range(0, q_seq_len, block_q):
        for j in range(0, kv_seq_len, block_k):
            rows = np.arange(i, i + block_q, dtype=np.int32)
            cols = np.arange(j, j + block_k, dtype=np.int32)
            if not np.asarray(mask_fn(rows[:, None], cols[None, :])).any():
                out[i // block_q, j // block_k] = False
    return out


def build_sliding_window_mask(
    *, q_seq_len: int, kv_seq_len: int, block_q: int, block_k: int, sliding_window_size: int
) -> np.ndarray:
    """flash_attention/common.py:83-104."""
    nq = -(-q_seq_len // block_q)
    nk = -(-kv_seq_len // block_k)
    out = np.tri(nq, nk, dtype=np.bool_)
    for i in range(0, q_seq_len, block_q):
        for j in range(0, kv_seq_len, block_k):
            if i - (j + block_k - 1) > sliding_window_size:
                out[i // block_q, j // block_k] = False
    return out


# ----------------------------------------------------------------------------------------------
# Seeded synthetic inputs for the BASELINE configurations.
# ----------------------------------------------------------------------------------------------


def normal_tensor(seed: int, shape, dtype=torch.float32) -> torch.Tensor:
    """iid N(0,1) from numpy's default_rng(seed), generated in fp32 then rounded to `dtype`."""
    x = np.random.default_rng(seed).standard_normal(size=shape, dtype=np.float32)
    return torch.from_numpy(x).to(dtype)


def packed_segment_ids(seed: int, batch: int, seq_len: int, max_docs: int = 6) -> torch.Tensor:
    """Per row: n ~ U{1..max_docs} documents, n-1 distinct sorted cut points uniform in [1, T-1];
    ids are the 1-based document index (0 is the padding id, flash_attention/common.py:618-620)."""
    rng = np.random.default_rng(seed)
    out = np.zeros((batch, seq_len), dtype=np.int32)
    for b in range(batch):
        n = int(rng.integers(1, max_docs + 1))
        cuts = np.sort(rng.choice(np.arange(1, seq_len), size=n - 1, replace=False)) if n > 1 else []
        ids = np.ones(seq_len, dtype=np.int32)
        for c in cuts:
            ids[c:] += 1
        out[b] = ids
    return torch.from_numpy(out)


def paged_inputs(seed: int, *, batch: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 page_size: int, pages_per_seq: int, min_len: int, max_len: int,
                 dtype=torch.bfloat16):
    """q [B,1,Hq,D], K/V pools [Hkv, B*pages_per_seq, page, D], page_tables [B, pages_per_seq]
    (a seeded permutation of all pool pages, as flash_attention/test_utils.py:64-66), lengths [B]."""
    total = batch * pages_per_seq
    q = normal_tensor(seed, (batch, 1, num_heads, head_dim), dtype)
    k = normal_tensor(seed + 1, (num_kv_heads, total, page_size, head_dim), dtype)
    v = normal_tensor(seed + 2, (num_kv_heads, total, page_size, head_dim), dtype)
    lengths = torch.from_numpy(
        np.random.default_rng(seed + 5).integers(min_len, max_len + 1, size=batch).astype(np.int32)
    )
    perm = np.random.default_rng(seed + 6).permutation(total).astype(np.int32)
    page_tables = torch.from_numpy(perm).reshape(batch, pages_per_seq)
    return q, k, v, page_tables, lengths


def count_unmasked_pairs(mask: MaskSpec, batch: int, q_len: int, kv_len: int, row_block: int = 1024) -> int:
    """Exact number of (b, q, k) pairs the mask keeps (dense bias ignored)."""
    total = 0
    for t0 in range(0, q_len, row_block):
        t1 = min(q_len, t0 + row_block)
        keep = mask.keep_rows(t0, t1, q_len, kv_len)
        if keep is None:
            total += batch * (t1 - t0) * kv_len
        else:
            n = int(keep.sum())
            total += n * (batch // keep.shape[0])
    return total


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a = a.to(torch.float64)
    b = b.to(torch.float64)
    return float((a - b).norm() / max(b.norm().item(), 1e-30))


def max_abs(a: torch.Tensor, b: torch.Tensor) -> float:
    return float((a.to(torch.float64) - b.to(torch.float64)).abs().max())
