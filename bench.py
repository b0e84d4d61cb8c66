"""Benchmark of the MI355X attention kernel path (one GPU).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|c1|c2|c3|c4|c5|f32] [--no-cpu-baseline]

The headline workload (BASELINE.json configs[1], "C2") is causal GQA flash attention forward +
backward, bf16, batch 4, 32 query heads / 8 kv heads, seq 4096, head_dim 128: a step is one forward
plus one backward over one synthetic batch already resident in HBM, obtained the way a caller of the
library obtains them: `flash_attention_implementation("gpu", ...)` with the default configuration, the
returned kernel object applied to the batch, `torch.autograd.grad` with a given dO (`c_abi_ms_per_step`
in the same object is the same pair of C-ABI calls with buffers allocated once).  The default
configuration keeps dS in the backward's workspace when that workspace fits a sixteenth of the
device's memory (C2: 2.15 GB, C3: 8.7 GB) and recomputes dS in the dQ kernel when it does not (C5:
69 GB); `backward` and `backward_chosen_by` say which ran.  `c2_recompute` / `c3_recompute` /
`c5_ds_workspace` in the same line are the same steps with the other backward forced through
`backend_overrides` (`--recompute` / `--ds-workspace` force it for the headline).
The paged-decode half of the metric (configs[3], "C4") is measured in the same run and reported in
the `paged_decode` object of the same JSON line.  With the default `--workload all` the line also
carries `c1` (configs[0]: the fp32 case the reference itself runs on CPU), `f32_row` (the fp32 row of the
reference's own kernel benchmark, forward and backward), `c3` (sliding window +
packed segments) and `c5` (one GPU's share of a 32768-token sequence), each with its own `roofline`
and `cpu_baseline`.

Inputs follow one seeding scheme, the same the parity tests use: numpy `default_rng(seed)`,
`standard_normal` in fp32, rounded to the element type; q = seed 0, k = 1, v = 2, dO = 3, segment
ids = 4, decode lengths = 5, page permutation = 6.

Prints ONE JSON line.  `value` = algorithmic TFLOP/s of fwd+bwd (4*B*Hq*T^2*D/2 forward, 2.5x that
backward; with segment ids the exact count of unmasked (query, key) pairs replaces T^2/2).
`roofline` describes the dominant kernel (the dK/dV backward kernel), timed with device events
around its own launches on the stream it runs on.  `cpu_baseline` times the CPU oracle
(oracle/ref_attention.py, a restatement of the reference's XLA attention) on a bounded slice of the
same workload on this machine's host cores.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
MFMA_F32_PEAK_TFLOPS = 157.3    # MI355X dense fp32 matrix
HBM_PEAK_GBS = 8000.0           # MI355X HBM3E

# HBM bytes per launch of each workload's dominant kernel come from profiles/traffic.json, which is
# written next to the rocprofv3 --pmc summaries it is taken from (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0,
# in KiB; the factors are what the same counters read for a plain 1 GiB copy kernel,
# `--calibrate-copy`): the run that prints them does not read the counters itself.
def _load_traffic():
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


TRAFFIC = _load_traffic()

METRIC = "flash-attn fwd+bwd TFLOP/s; paged-decode HBM GB/s (% roofline), 1 MI355X"


def normal_tensor(seed, shape, dtype, device):
    """iid N(0,1) from numpy's default_rng(seed), generated in fp32, rounded to `dtype`, moved to the GPU
    in slices (bounds the host staging buffer)."""
    rng = np.random.default_rng(seed)
    out = torch.empty(shape, dtype=dtype, device=device)
    flat = out.view(-1)
    n, step = flat.numel(), 1 << 26
    for i in range(0, n, step):
        m = min(step, n - i)
        flat[i:i + m] = torch.from_numpy(rng.standard_normal(size=m, dtype=np.float32)).to(device).to(dtype)
    return out


def _events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def _time_region(fn, steps, warmup, settle_s=0.0):
    """Runs warmup + steps calls of fn; returns ms per step from device events on torch's current
    stream (the stream every C-ABI call is enqueued on).  `settle_s`: ahead of the warm-up steps, keep
    calling fn for that long, untimed: after the idle stretch in which the inputs were generated the
    power manager takes tens of milliseconds to bring the clocks to where a running job has them (the
    first 20 steps after 5 warm-up steps measured 3 % slower than every later 20)."""
    if settle_s > 0.0:
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < settle_s:
            for _ in range(4):
                fn()
            torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = _events(2)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def _flash_workload(name):
    if name == "c2":
        return dict(name="c2", label="C2: causal GQA flash fwd+bwd, bf16, B4 Hq32/Hkv8 T4096 D128",
                    B=4, T=4096, Hq=32, Hkv=8, D=128, mask="causal", window=0, seg=False)
    if name == "c3":
        return dict(name="c3", label="C3: sliding-window(4096) causal MHA + segment ids fwd+bwd, bf16, B8 H16 T8192 D128",
                    B=8, T=8192, Hq=16, Hkv=16, D=128, mask="sliding", window=4096, seg=True)
    if name == "c5":
        return dict(name="c5", label="C5: long-context causal GQA fwd+bwd, bf16, B1 Hq64/Hkv8 T32768 D128",
                    B=1, T=32768, Hq=64, Hkv=8, D=128, mask="causal", window=0, seg=False)
    raise ValueError(name)


def packed_segment_ids(seed, batch, seq_len, max_docs=6):
    """Per row: n ~ U{1..max_docs} documents split at n-1 distinct uniform cut points; ids are the
    1-based document index (id 0 is reserved for padding)."""
    rng = np.random.default_rng(seed)
    out = np.ones((batch, seq_len), dtype=np.int32)
    for b in range(batch):
        n = int(rng.integers(1, max_docs + 1))
        if n > 1:
            for c in np.sort(rng.choice(np.arange(1, seq_len), size=n - 1, replace=False)):
                out[b, c:] += 1
    return torch.from_numpy(out)


def count_pairs(seg, window):
    """Exact number of (batch, query, key) pairs kept by sliding-window-causal AND equal segment."""
    B, T = seg.shape
    pos = torch.arange(T, device=seg.device)
    total = 0
    for t0 in range(0, T, 1024):
        qp = pos[t0:t0 + 1024, None]
        keep = (qp >= pos[None, :]) & (qp - pos[None, :] <= window)
        keep = keep[None] & (seg[:, t0:t0 + 1024, None] == seg[:, None, :])
        total += int(keep.sum())
    return total


def _traffic(name):
    t = TRAFFIC.get(name)
    return (None, None) if t is None else (t["bytes"], t["source"])


def _dispatch_bias(cfg, seg, T, dev):
    """The attention bias a layer would hand to the dispatch for this workload."""
    from axlearn_amd import attention_bias as ab

    pos = dict(target_positions=torch.arange(T, device=dev)[None], source_positions=torch.arange(T, device=dev)[None])
    parts = []
    if cfg["mask"] == "causal":
        parts.append(ab.CausalAttentionBias(**pos))
    elif cfg["mask"] == "sliding":
        parts.append(ab.SlidingWindowAttentionBias(ab.sliding_window_causal_mask(cfg["window"]),
                                                   sliding_window_size=cfg["window"], **pos))
    if seg is not None:
        parts.append(ab.SegmentIdAttentionBias(seg))
    return ab.CompositeAttentionBias(parts)


def bench_flash(cfg, steps, warmup, cpu_baseline):
    """One fwd+bwd step = what a caller of `flash_attention_implementation("gpu", ...)` gets: the
    returned kernel object applied to the batch, then autograd's backward with a given dO.
    cfg["ds_workspace"]: None = the plugin's default (dS workspace when it fits the default limit, a
    sixteenth of the device's memory - whole, or the dS of a few kv heads at a time), True / False =
    forced through backend_overrides (True: the whole dS at once)."""
    from axlearn_amd import ops
    from axlearn_amd.flash_attention.utils import flash_attention_implementation

    dev = torch.device("cuda:0")
    B, T, Hq, Hkv, D = cfg["B"], cfg["T"], cfg["Hq"], cfg["Hkv"], cfg["D"]
    bf = torch.bfloat16
    q = normal_tensor(0, (B, T, Hq, D), bf, dev).requires_grad_(True)
    k = normal_tensor(1, (B, T, Hkv, D), bf, dev).requires_grad_(True)
    v = normal_tensor(2, (B, T, Hkv, D), bf, dev).requires_grad_(True)
    do = normal_tensor(3, (B, T, Hq, D), bf, dev)
    seg = None
    pairs = None
    if cfg["seg"]:
        seg = packed_segment_ids(4, B, T).to(dev)
        pairs = count_pairs(seg, cfg["window"])
    mask_kind = {"none": ops.MASK_NONE, "causal": ops.MASK_CAUSAL, "sliding": ops.MASK_SLIDING_WINDOW}[cfg["mask"]]
    forced = cfg.get("ds_workspace")
    slice_heads = 0   # kv heads whose dS the workspace holds at a time (0: all)
    if forced is None:
        spill, slice_heads = ops.select_ds_slice(q, k, mask_kind=mask_kind, segment_ids=seg)
        chosen = "default config (by workspace size)"
    else:
        spill = bool(forced)
        chosen = f"backend_overrides bwd_ds_workspace={spill}"
    ws_need, _ = ops.flash_bwd_ds_workspace_bytes(q, k, mask_kind=mask_kind, segment_ids=seg,
                                                  ds_slice_kv_heads=slice_heads)
    bias = _dispatch_bias(cfg, seg, T, dev)
    impl = flash_attention_implementation(
        "gpu", query=q, key=k, value=v, bias=bias, softmax_scale=D ** -0.5,
        backend_overrides=None if forced is None else dict(bwd_ds_workspace=spill))
    if impl is None:
        sys.exit("bench.py: the dispatch found no kernel for " + cfg["label"])
    batch = dict(query=q, key=k, value=v, bias=bias)

    def step():
        # gradients handed back to the caller, as they are to the layer below attention in a model (a
        # .backward() into leaf tensors would add a copy of every gradient: autograd clones what it
        # accumulates into a leaf)
        torch.autograd.grad(impl.fn(batch), (q, k, v), do)

    ms_step = _time_region(step, steps, warmup, settle_s=0.25)
    # The same kernels through the C ABI with buffers allocated once (no allocator, no autograd).
    qd, kd, vd = q.detach(), k.detach(), v.detach()
    kw = dict(softmax_scale=D ** -0.5, mask_kind=mask_kind, sliding_window=cfg["window"], segment_ids=seg)
    bufs = ops.flash_bwd_buffers(qd, kd, vd, mask_kind=mask_kind, ds_workspace=spill, segment_ids=seg,
                                 ds_slice_kv_heads=slice_heads)
    kw_b = dict(kw, ds_workspace=spill, ds_slice_kv_heads=slice_heads)
    out, lse = ops.flash_fwd(qd, kd, vd, **kw)

    def abi_step():
        o, l = ops.flash_fwd(qd, kd, vd, **kw)
        ops.flash_bwd(qd, kd, vd, o, l, do, buffers=bufs, **kw_b)

    ms_abi = _time_region(abi_step, steps, 2)
    # Per-kernel durations, each kernel timed over its own launches (device events on the stream the
    # launches go to).  With the dS workspace the dq phase reads what the dK/dV phase before it left.
    ms_fwd = _time_region(lambda: ops.flash_fwd(qd, kd, vd, **kw), steps, 1)
    ms_delta = _time_region(lambda: ops.flash_bwd(qd, kd, vd, out, lse, do, buffers=bufs, phases=1, **kw_b), steps, 1)
    n_slices = 1
    if slice_heads:
        # The dK/dV and dQ kernels run once per slice of kv heads, every launch on the same amount of work:
        # one slice's launch of each is timed on its own (the first slice's heads as a problem of their
        # own, which is what the library enqueues), the step holds n_slices of them.
        n_slices = -(-Hkv // slice_heads)
        hq_s = slice_heads * (Hq // Hkv)
        qs, ks, vs, dos, outs = qd[:, :, :hq_s], kd[:, :, :slice_heads], vd[:, :, :slice_heads], do[:, :, :hq_s], out[:, :, :hq_s]
        lses = lse[:, :hq_s].contiguous()
        kw_s = dict(kw, ds_workspace=True)
        bufs_s = ops.flash_bwd_buffers(qs, ks, vs, mask_kind=mask_kind, ds_workspace=True, segment_ids=seg)
        ops.flash_bwd(qs, ks, vs, outs, lses, dos, buffers=bufs_s, **kw_s)
        ms_dkdv = n_slices * _time_region(
            lambda: ops.flash_bwd(qs, ks, vs, outs, lses, dos, buffers=bufs_s, phases=2, **kw_s), steps, 1)
        ms_dq = n_slices * _time_region(
            lambda: ops.flash_bwd(qs, ks, vs, outs, lses, dos, buffers=bufs_s, phases=4, **kw_s), steps, 1)
        del bufs_s
    else:
        ms_dkdv = _time_region(lambda: ops.flash_bwd(qd, kd, vd, out, lse, do, buffers=bufs, phases=2, **kw_b), steps, 1)
        ms_dq = _time_region(lambda: ops.flash_bwd(qd, kd, vd, out, lse, do, buffers=bufs, phases=4, **kw_b), steps, 1)

    if pairs is None:
        gemm = 2.0 * B * Hq * (T * T / 2.0) * D  # one [T,T,D] causal GEMM (the 1/2 convention)
    else:
        gemm = 2.0 * Hq * pairs * D               # exact count of unmasked (q,k) pairs
    fl_fwd, fl_bwd = 2 * gemm, 5 * gemm
    fl_dkdv, fl_dq = 4 * gemm, 1 * gemm           # S, dP, dV, dK | dQ
    tf = lambda fl, ms: fl / (ms * 1e-3) / 1e12
    dq_name = "flash_bwd_dq_stream_kernel" if spill else "flash_bwd_dq_ring_kernel"
    traffic, traffic_src = _traffic(cfg["name"] + ("" if spill else "_recompute"))
    result = dict(
        workload=cfg["label"], value=tf(fl_fwd + fl_bwd, ms_step), unit="TFLOP/s", ms_per_step=ms_step,
        entry="flash_attention_implementation('gpu', ...).fn(batch) + torch.autograd.grad(out, (q, k, v), dO)",
        backward=("dS workspace: delta, dK/dV (stores dS), dq = dS k"
                  + (f", the last two once per slice of {slice_heads} kv heads ({n_slices} slices)" if slice_heads else "")
                  if spill else "dQ (recomputes dS, computes delta), dK/dV"),
        backward_chosen_by=chosen, ds_workspace_bytes=ws_need if spill else 0, ds_slice_kv_heads=slice_heads,
        c_abi_ms_per_step=ms_abi,
        kernels={
            "flash_fwd_kernel": dict(ms=ms_fwd, tflops=tf(fl_fwd, ms_fwd), algorithmic_tflop=fl_fwd / 1e12),
            "bwd_delta_kernel": dict(ms=ms_delta, in_step=spill),
            "flash_bwd_dkdv_kernel": dict(ms=ms_dkdv, tflops=tf(fl_dkdv, ms_dkdv), algorithmic_tflop=fl_dkdv / 1e12),
            dq_name: dict(ms=ms_dq, tflops=tf(fl_dq, ms_dq), algorithmic_tflop=fl_dq / 1e12),
        },
        roofline=dict(
            kernel="flash_bwd_dkdv_kernel", bound="mfma", achieved=tf(fl_dkdv, ms_dkdv),
            peak=MFMA_BF16_PEAK_TFLOPS, unit="TFLOP/s", frac=tf(fl_dkdv, ms_dkdv) / MFMA_BF16_PEAK_TFLOPS,
            traffic=traffic, traffic_source=traffic_src,
        ),
        step_frac_of_mfma_peak=tf(fl_fwd + fl_bwd, ms_step) / MFMA_BF16_PEAK_TFLOPS,
    )
    if pairs is not None:
        result["unmasked_pairs"] = pairs
    if cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_flash(cfg)
    del q, k, v, qd, kd, vd, do, out, lse, bufs, batch, impl
    torch.cuda.empty_cache()
    return result


def cpu_baseline_flash(cfg, budget_s=8.0):
    """Times the oracle's fwd+bwd (reverse-mode autodiff of the ReferenceMHA restatement, fp32 math
    on bf16-rounded inputs) on a slice of the workload: batch element 0, kv heads [0, nkv)."""
    from oracle import ref_attention as ref

    T, Hq, Hkv, D = cfg["T"], cfg["Hq"], cfg["Hkv"], cfg["D"]
    G = Hq // Hkv
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    nkv = 1
    t_cap = min(T, 4096)  # rows [0, t_cap) of the causal problem: a self-contained causal sub-problem
    q = ref.normal_tensor(0, (1, t_cap, nkv * G, D), torch.bfloat16)
    k = ref.normal_tensor(1, (1, t_cap, nkv, D), torch.bfloat16)
    v = ref.normal_tensor(2, (1, t_cap, nkv, D), torch.bfloat16)
    do = ref.normal_tensor(3, (1, t_cap, nkv * G, D), torch.bfloat16)
    seg = ref.packed_segment_ids(4, 1, t_cap) if cfg["seg"] else None
    spec = ref.MaskSpec(causal=cfg["mask"] == "causal",
                        sliding_window=cfg["window"] if cfg["mask"] == "sliding" else None, segment_ids=seg)
    t0 = time.perf_counter()
    reps = 0
    while True:
        ref.reference_mha_grads(q, k, v, do, spec, softmax_scale=D ** -0.5, row_block=512, dtype=torch.float32)
        reps += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or reps >= 64:
            break
    pairs = ref.count_unmasked_pairs(spec, 1, t_cap, t_cap) if cfg["seg"] else t_cap * t_cap / 2.0
    flops = 7.0 * 2.0 * (nkv * G) * pairs * D  # fwd (2 GEMMs) + bwd (5 GEMMs), algorithmic
    return dict(
        value=flops * reps / dt / 1e12, unit="TFLOP/s", cores=cores, kind="port",
        sample=f"oracle fwd+bwd (torch-CPU autodiff, fp32) on batch 0, {nkv} kv head ({nkv * G} query heads), "
               f"rows 0..{t_cap - 1}; {reps} repetitions in {dt:.1f} s",
    )


def bench_f32_row(steps, warmup):
    """The fp32 row of the reference's own kernel benchmark (gpu_attention_benchmark.py:55-59, :93-97):
    causal MHA, batch 2, 32 heads, 4096 tokens, head_dim 128, forward and backward through the C ABI.  A
    side line: fp32 products are formed from bf16 parts on the bf16 matrix instruction."""
    from axlearn_amd import ops

    dev = torch.device("cuda:0")
    B, T, H, D = 2, 4096, 32, 128
    q, k, v, do = (normal_tensor(s, (B, T, H, D), torch.float32, dev) for s in (0, 1, 2, 3))
    kw = dict(softmax_scale=D ** -0.5, mask_kind=ops.MASK_CAUSAL)
    out, lse = ops.flash_fwd(q, k, v, **kw)
    bufs = ops.flash_bwd_buffers(q, k, v, mask_kind=ops.MASK_CAUSAL)
    n = max(3, steps // 4)
    ms_fwd = _time_region(lambda: ops.flash_fwd(q, k, v, **kw), n, min(warmup, 2))
    ms_bwd = _time_region(lambda: ops.flash_bwd(q, k, v, out, lse, do, buffers=bufs, **kw), n, min(warmup, 2))
    fl_fwd = 4.0 * B * H * T * T * D / 2.0
    return dict(
        workload="reference benchmark row: causal MHA fwd / bwd, fp32, B2 H32 T4096 D128",
        arithmetic="fp32 operands as three bf16 parts each, six bf16 MFMA partial products per product, fp32 accumulation",
        fwd_ms=ms_fwd, bwd_ms=ms_bwd, fwd_tflops=fl_fwd / (ms_fwd * 1e-3) / 1e12,
        bwd_tflops=2.5 * fl_fwd / (ms_bwd * 1e-3) / 1e12, fp32_mfma_peak_tflops=MFMA_F32_PEAK_TFLOPS,
        kernels=["flash_fwd_f32x_kernel", "flash_bwd_dkdv_f32x_kernel", "flash_bwd_dq_f32x_kernel"],
    )


def bench_c1(steps, warmup, cpu_baseline):
    """C1 (configs[0]): causal MHA forward, fp32, B2 H4 T512 D64, scale 1/8.  The CPU oracle is the
    subject (timed in full); the fp32 forward kernel is timed, and checked against it, beside it."""
    from axlearn_amd import ops

    dev = torch.device("cuda:0")
    B, T, H, D = 2, 512, 4, 64
    q, k, v = (normal_tensor(s, (B, T, H, D), torch.float32, dev) for s in (0, 1, 2))
    kw = dict(softmax_scale=0.125, mask_kind=ops.MASK_CAUSAL)
    ms = _time_region(lambda: ops.flash_fwd(q, k, v, **kw), max(steps, 50), warmup)
    flops = 4.0 * B * H * T * T * D / 2.0
    tfl = flops / (ms * 1e-3) / 1e12
    res = dict(
        workload="C1: causal MHA forward, fp32, B2 H4 T512 D64", value=tfl, unit="TFLOP/s", ms_per_step=ms,
        algorithmic_gflop=flops / 1e9,
        arithmetic="fp32 operands as three bf16 parts each, six bf16 MFMA partial products per product, fp32 accumulation",
        executed_tflops=6.0 * tfl, fp32_mfma_peak_tflops=MFMA_F32_PEAK_TFLOPS,
        roofline=dict(kernel="flash_fwd_f32x_kernel", bound="mfma", achieved=tfl, peak=MFMA_BF16_PEAK_TFLOPS,
                      unit="TFLOP/s", frac=tfl / MFMA_BF16_PEAK_TFLOPS, traffic=None,
                      traffic_source="not measured: 32 workgroups, 0.27 GFLOP, bound by launch latency"),
    )
    if cpu_baseline:
        from oracle import ref_attention as ref

        cores = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(cores)
        qc, kc, vc = q.cpu(), k.cpu(), v.cpu()
        spec = ref.MaskSpec(causal=True)
        want = ref.reference_mha(qc, kc, vc, spec, softmax_scale=0.125)
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < 2.0:
            ref.reference_mha(qc, kc, vc, spec, softmax_scale=0.125, mode="faithful")
            reps += 1
        dt = time.perf_counter() - t0
        out, _ = ops.flash_fwd(q, k, v, **kw)
        res["max_abs_vs_oracle"] = float((out.cpu().double() - want.double()).abs().max())
        res["cpu_baseline"] = dict(
            value=flops * reps / dt / 1e12, unit="TFLOP/s", ms_per_step=dt / reps * 1e3, cores=cores, kind="port",
            sample=f"oracle ReferenceMHA restatement (fp32, the reference's rounding points), the whole of C1, "
                   f"{reps} repetitions in {dt:.1f} s",
        )
    return res


def bench_paged_decode(steps, warmup, cpu_baseline):
    """C4: B64, Hq32/Hkv8, D128, page 16, pool of 64*2048 pages, lengths U[512, 32768]."""
    from axlearn_amd import ops

    dev = torch.device("cuda:0")
    B, Hq, Hkv, D, page, pps = 64, 32, 8, 128, 16, 2048
    P = B * pps
    bf = torch.bfloat16
    kp = normal_tensor(1, (Hkv, P, page, D), bf, dev)
    vp = normal_tensor(2, (Hkv, P, page, D), bf, dev)
    q = normal_tensor(0, (B, Hq, D), bf, dev)
    lengths_cpu = torch.from_numpy(np.random.default_rng(5).integers(512, 32769, size=B).astype(np.int32))
    tables_cpu = torch.from_numpy(np.random.default_rng(6).permutation(P).astype(np.int32)).reshape(B, pps)
    lengths, tables = lengths_cpu.to(dev), tables_cpu.to(dev)
    out = torch.empty((B, Hq, D), device=dev, dtype=bf)
    ws = torch.empty((ops.paged_decode_workspace_bytes(B, Hq, Hkv, D, pps),), device=dev, dtype=torch.uint8)
    scale = D ** -0.5
    # The timed call is what a caller whose scratch memory comes from an allocator per call (XLA) gets:
    # the library zeroes the work counter of a workspace it knows nothing about (one extra one-thread
    # launch).  A serving loop that keeps one workspace sets AXL_DECODE_WORKSPACE_REUSED from its second
    # call on and launches the split and merge kernels only: reported beside it.
    fn = lambda: ops.paged_decode(q, kp, vp, tables, lengths, softmax_scale=scale, workspace=ws, out=out)
    ms = _time_region(fn, steps, warmup, settle_s=0.1)
    fn_reused = lambda: ops.paged_decode(q, kp, vp, tables, lengths, softmax_scale=scale, workspace=ws, out=out,
                                         workspace_reused=True)
    ms_reused = _time_region(fn_reused, steps, 2)
    # The fixed work decomposition (AXL_DECODE_DETERMINISTIC: bit-reproducible results).
    fn_det = lambda: ops.paged_decode(q, kp, vp, tables, lengths, softmax_scale=scale, workspace=ws, out=out,
                                      deterministic=True)
    ms_det = _time_region(fn_det, steps, 2)
    # The same sequences in 64-token pages (one of the page sizes the reference admits besides 16): the
    # pools are re-viewed, so every 64-token page is four of the old ones that happen to be adjacent, and
    # the table is a permutation of those.
    kp64, vp64 = kp.view(Hkv, P // 4, 64, D), vp.view(Hkv, P // 4, 64, D)
    tables64 = torch.from_numpy(np.random.default_rng(6).permutation(P // 4).astype(np.int32)).reshape(B, pps // 4).to(dev)
    fn64 = lambda: ops.paged_decode(q, kp64, vp64, tables64, lengths, softmax_scale=scale, workspace=ws, out=out)
    ms64 = _time_region(fn64, steps, 2)
    live64 = int(((lengths_cpu.long() + 63) // 64).sum())
    bytes64 = live64 * 64 * Hkv * D * 2 * 2 + live64 * 4 + 2 * B * Hq * D * 2
    live_pages = int(((lengths_cpu.long() + page - 1) // page).sum())
    # Algorithmic bytes: every live K and V page once, its page-table entry, q and out.
    algo_bytes = live_pages * page * Hkv * D * 2 * 2 + live_pages * 4 + 2 * B * Hq * D * 2
    gbs = algo_bytes / (ms * 1e-3) / 1e9
    traffic, traffic_src = _traffic("c4")
    res = dict(
        workload="C4: paged decode, bf16, B64 Hq32/Hkv8 D128, page 16, ctx U[512,32768]",
        value=gbs, unit="GB/s", ms_per_step=ms, algorithmic_gb=algo_bytes / 1e9,
        workspace_reused=dict(ms_per_step=ms_reused, value=algo_bytes / (ms_reused * 1e-3) / 1e9, unit="GB/s"),
        deterministic=dict(ms_per_step=ms_det, value=algo_bytes / (ms_det * 1e-3) / 1e9, unit="GB/s"),
        page_size_64=dict(ms_per_step=ms64, value=bytes64 / (ms64 * 1e-3) / 1e9, unit="GB/s",
                          algorithmic_gb=bytes64 / 1e9),
        roofline=dict(kernel="decode_split_kernel", bound="hbm", achieved=gbs, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=gbs / HBM_PEAK_GBS, traffic=traffic, traffic_source=traffic_src),
    )
    if cpu_baseline:
        from oracle import ref_attention as ref

        nb = 32  # sequences timed on the CPU
        cores = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(cores)
        kc, vc = kp.cpu(), vp.cpu()
        qc = q[:nb].cpu().unsqueeze(1)
        t0 = time.perf_counter()
        ref.reference_decode(qc, kc, vc, lengths_cpu[:nb], softmax_scale=scale, page_tables=tables_cpu[:nb], mode="faithful")
        dt = time.perf_counter() - t0
        nbytes = int(((lengths_cpu[:nb].long() + page - 1) // page).sum()) * page * Hkv * D * 2 * 2
        res["cpu_baseline"] = dict(
            value=nbytes / dt / 1e9, unit="GB/s", cores=cores, kind="port",
            sample=f"oracle ReferenceMHA restatement (page gather + dense attention) on sequences 0..{nb - 1}, {dt:.2f} s",
        )
        del kc, vc
    del kp, vp
    torch.cuda.empty_cache()
    return res


def calibrate_mfma(n=8192, reps=20):
    """What the matrix cores of this machine sustain on a plain library GEMM (torch.matmul, bf16,
    n^3) with N(0,1) operands and with all-zero operands: the clock is set by the power the operands'
    bit activity draws, so the two differ, and the first is the practical ceiling for any kernel whose
    MFMAs see random data.  Calibration only, like --calibrate-copy; no part of the measured path."""
    dev = torch.device("cuda:0")
    out = {}
    for kind in ("normal", "zeros"):
        if kind == "normal":
            a = normal_tensor(7, (n, n), torch.bfloat16, dev)
            b = normal_tensor(8, (n, n), torch.bfloat16, dev)
        else:
            a = torch.zeros((n, n), dtype=torch.bfloat16, device=dev)
            b = torch.zeros((n, n), dtype=torch.bfloat16, device=dev)
        c = torch.empty((n, n), dtype=torch.bfloat16, device=dev)
        ms = _time_region(lambda: torch.matmul(a, b, out=c), reps, 10)
        out[f"gemm_bf16_{n}_{kind}_tflops"] = 2.0 * n ** 3 / (ms * 1e-3) / 1e12
        del a, b, c
    out["note"] = "torch.matmul (hipBLASLt) bf16 GEMM, calibration of the power-limited matrix-core rate"
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all", choices=["all", "c1", "c2", "c3", "c4", "c5", "f32"],
                    help="all: headline C2 + C4, with C1, C3 and C5 as extra keys of the same line")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true", help="skip the paged-decode half of the metric")
    ap.add_argument("--recompute", action="store_true",
                    help="force the backward whose dQ kernel recomputes dS (no dS workspace)")
    ap.add_argument("--ds-workspace", action="store_true",
                    help="force the backward that keeps dS in its workspace, whatever its size")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (known traffic) for scaling rocprofv3 byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU only (no collectives, no sharding); use --gpus 1.")
    if int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: launched with WORLD_SIZE > 1; this build runs on one GPU only.")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP kernels have no CPU path.")
    cpu_base = not args.no_cpu_baseline
    if args.calibrate_copy:
        # A plain elementwise copy kernel that reads exactly 1 GiB and writes exactly 1 GiB.
        src = torch.ones((1 << 28,), device="cuda:0", dtype=torch.float32)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 0.0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    line = dict(metric=METRIC, n_gpus=1, steps=args.steps, warmup=args.warmup, higher_is_better=True,
                scaling="weak", vs_baseline=None, dtype="bf16", data="synthetic")
    if args.workload == "c4":
        dec = bench_paged_decode(args.steps, args.warmup, cpu_base)
        line.update(value=dec["value"], unit="GB/s", ms_per_step=dec["ms_per_step"],
                    config=dict(workload=dec["workload"]), roofline=dec["roofline"])
        if "cpu_baseline" in dec:
            line["cpu_baseline"] = dec["cpu_baseline"]
        line["paged_decode"] = dec
    elif args.workload == "f32":
        res = bench_f32_row(args.steps, args.warmup)
        line.update(value=res["fwd_tflops"], unit="TFLOP/s", ms_per_step=res["fwd_ms"], dtype="f32",
                    config=dict(workload=res["workload"]), f32_row=res)
    elif args.workload == "c1":
        res = bench_c1(args.steps, args.warmup, cpu_base)
        line.update(value=res["value"], unit="TFLOP/s", ms_per_step=res["ms_per_step"], dtype="f32",
                    config=dict(workload=res["workload"]), roofline=res["roofline"])
        if "cpu_baseline" in res:
            line["cpu_baseline"] = res["cpu_baseline"]
        line["c1"] = res
    else:
        cfg = _flash_workload("c2" if args.workload == "all" else args.workload)
        forced = False if args.recompute else (True if args.ds_workspace else None)
        cfg = dict(cfg, ds_workspace=forced)
        res = bench_flash(cfg, args.steps, args.warmup, cpu_base)
        line.update(value=res["value"], unit="TFLOP/s", ms_per_step=res["ms_per_step"],
                    config=dict(workload=cfg["label"], batch=cfg["B"], seq_len=cfg["T"], num_q_heads=cfg["Hq"],
                                num_kv_heads=cfg["Hkv"], head_dim=cfg["D"], mask=cfg["mask"], window=cfg["window"],
                                segment_ids=cfg["seg"], entry=res["entry"], backward=res["backward"],
                                backward_chosen_by=res["backward_chosen_by"]),
                    roofline=res["roofline"], kernels=res["kernels"], c_abi_ms_per_step=res["c_abi_ms_per_step"],
                    step_frac_of_mfma_peak=res["step_frac_of_mfma_peak"])
        if "unmasked_pairs" in res:
            line["unmasked_pairs"] = res["unmasked_pairs"]
        if "cpu_baseline" in res:
            line["cpu_baseline"] = res["cpu_baseline"]
        if not args.no_decode:
            line["paged_decode"] = bench_paged_decode(args.steps, args.warmup, cpu_base)
        if args.workload == "all":
            # The other BASELINE configs, fewer repetitions: they are reported, not the headline.
            def other(name, first, n_steps, n_warm):
                # the same step with the backward the default did not pick, forced through backend_overrides
                took_ds = first["backward"].startswith("dS workspace")
                key = name + ("_recompute" if took_ds else "_ds_workspace")
                line[key] = bench_flash(dict(_flash_workload(name), ds_workspace=not took_ds), n_steps, n_warm, False)

            other("c2", res, args.steps, args.warmup)
            line["machine"] = calibrate_mfma()
            line["c1"] = bench_c1(args.steps, args.warmup, cpu_base)
            line["f32_row"] = bench_f32_row(args.steps, args.warmup)
            line["c3"] = bench_flash(dict(_flash_workload("c3"), ds_workspace=forced), max(5, args.steps // 2), 2, cpu_base)
            other("c3", line["c3"], max(5, args.steps // 2), 2)
            line["c5"] = bench_flash(dict(_flash_workload("c5"), ds_workspace=forced), max(3, args.steps // 4), 1, cpu_base)
            other("c5", line["c5"], max(3, args.steps // 4), 1)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
