"""Wall times of the MI355X attention kernels on the shapes of the reference's kernel benchmark.

Mirrors the sweeps of axlearn/common/flash_attention/gpu_attention_benchmark.py:318-375 (decode over
batch x context, decode over kv heads, decode with sliding windows, prefill forward and
forward + backward over batch, heads, sequence length, head dim and sliding windows; float16, causal
MHA unless stated, as `bench_flash_attention`, :208-262) and prints the same kind of table: one line
per combination, milliseconds per call.  The kernels are reached the way the reference's benchmark
reaches them: through the kernel classes' `is_supported` + `__call__` (`HipFlashAttention`,
`HipDecoding`), with the mask given as an attention bias.

Method, as the reference's `measure` (:163-206): every timed call is enqueued behind two large GEMMs, so
that the device events bracket device work and neither the launch latency of an idle GPU (25 us here,
more than the smallest decode calls take) nor this module's Python, which runs while the GEMMs do; the
time is the median of `--iters` such calls after `--warmup` calls (the reference reports one).
`--graph` captures the forward-only and decode calls once and times the replays instead (a replay has a
floor of 13 us here, whatever it holds).  `use_bwd=True` times the forward and the backward of `mean(out)`
together, which is what `jax.grad` of the forward computes.

Run: python -m axlearn_amd.flash_attention.hip_attention_benchmark [--quick] [--iters N]
"""

from __future__ import annotations

import argparse
import itertools
import statistics
from typing import Any, Optional

import torch

from axlearn_amd import attention_bias as ab
from axlearn_amd.flash_attention.hip_attention import HipFlashAttention
from axlearn_amd.flash_attention.hip_decoding import HipDecoding
from axlearn_amd.kv_cache import KVCache


def _bias(q_len: int, kv_len: int, sw_sz: int, query_offset: int, device) -> ab.BaseAttentionBias:
    # int32 positions, as jnp.arange gives the reference's benchmark
    pos = dict(
        target_positions=(torch.arange(q_len, device=device, dtype=torch.int32) + query_offset)[None],
        source_positions=torch.arange(kv_len, device=device, dtype=torch.int32)[None],
    )
    if sw_sz != -1:
        return ab.CompositeAttentionBias([
            ab.SlidingWindowAttentionBias(ab.sliding_window_causal_mask(sw_sz), sliding_window_size=sw_sz, **pos)
        ])
    return ab.CompositeAttentionBias([ab.CausalAttentionBias(**pos)])


def measure(fn, warmup: int, iters: int, graph: bool = False) -> float:
    """Median milliseconds of `fn()` over `iters` calls, timed with device events; with `graph` the
    call is captured once and its replays are timed.  Each timed call is enqueued while two large GEMMs
    still run ahead of it, so its launch is hidden and the events see device time only
    (gpu_attention_benchmark.py:163-206)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(warmup):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    if graph:
        captured = torch.cuda.CUDAGraph()
        with torch.cuda.graph(captured):
            fn()
        fn = captured.replay
        fn()
        torch.cuda.synchronize()
    x = torch.ones((8192, 8192), dtype=torch.float16, device="cuda")   # a GEMM of about a millisecond
    times = []
    for _ in range(iters):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(2):
            _ = x @ x
        start.record()
        fn()
        end.record()
        end.synchronize()
        times.append(start.elapsed_time(end))
    return statistics.median(times)


def bench_flash_attention(
    *,
    bs: int,
    num_heads: int,
    num_kv_heads: Optional[int],
    seq_len: int,
    per_head_dim: int,
    is_decode: bool,
    use_bwd: bool,
    sw_sz: int = -1,
    dtype=torch.float16,
    warmup: int = 3,
    iters: int = 10,
    graph: bool = False,
) -> float:
    if use_bwd and is_decode:
        raise ValueError("use_bwd and is_decode cannot both be true.")
    device = torch.device("cuda:0")
    num_kv_heads = num_kv_heads or num_heads
    q_len = 1 if is_decode else seq_len
    gen = torch.Generator(device=device).manual_seed(0)
    q = torch.randn((bs, q_len, num_heads, per_head_dim), generator=gen, device=device, dtype=dtype)
    k = torch.randn((bs, seq_len, num_kv_heads, per_head_dim), generator=gen, device=device, dtype=dtype)
    v = torch.randn((bs, seq_len, num_kv_heads, per_head_dim), generator=gen, device=device, dtype=dtype)
    bias = _bias(q_len, seq_len, sw_sz, seq_len - 1 if is_decode else 0, device)
    cls = HipDecoding if is_decode else HipFlashAttention
    fn = cls.default_config().set(softmax_scale=per_head_dim ** -0.5).instantiate()
    batch = dict(query=q, key=k, value=v, bias=bias)
    if not fn.is_supported(batch, kv_cache_type=KVCache if is_decode else None):
        raise ValueError(f"{cls.__name__} declines {bs=} {num_heads=} {num_kv_heads=} {seq_len=} {per_head_dim=}")
    if not use_bwd:
        with torch.no_grad():
            return measure(lambda: fn(batch), warmup, iters, graph)
    for x in (q, k, v):
        x.requires_grad_(True)

    def step():
        q.grad = k.grad = v.grad = None
        fn(batch).mean().backward()

    return measure(step, warmup, iters)


def _sweep(common: dict[str, Any], opts: dict[str, Any], **sweep: list[Any]) -> None:
    common = {k: v for k, v in common.items() if k not in sweep}
    print(", ".join(f"{k}={v}" for k, v in common.items()))
    print("{:<50}{:<14}".format("", "axlearn_amd"))
    for comb in itertools.product(*[[(k, v) for v in vs] for k, vs in sweep.items()]):
        ms = bench_flash_attention(**dict(comb), **common, **opts)
        print("{:<50}{:<14.6f}".format(",".join(f"{k}={v}" for k, v in comb), ms), flush=True)


def benchmark_decode(opts, quick: bool) -> None:
    common = dict(is_decode=True, use_bwd=False, bs=1, num_heads=8, num_kv_heads=8, seq_len=32 * 1024,
                  per_head_dim=128, sw_sz=-1)
    lens = [1024, 4096, 8192, 131072]
    _sweep(common, opts, bs=[1, 32] if quick else [1, 4, 8, 16, 32], seq_len=lens)
    _sweep(common, opts, bs=[1, 8], num_kv_heads=[1, 8])
    _sweep(common, opts, bs=[1, 8], seq_len=[131072], sw_sz=[-1, 4096, 16 * 1024])


def benchmark_prefill(opts, use_bwd: bool, quick: bool) -> None:
    common = dict(is_decode=False, use_bwd=use_bwd, bs=2, num_heads=32, num_kv_heads=None, seq_len=4096,
                  per_head_dim=128, sw_sz=-1)
    _sweep(common, opts, bs=[2, 4, 8])
    _sweep(common, opts, bs=[2] if quick else [2, 4, 8], dtype=[torch.float32])
    if not quick:
        _sweep(common, opts, num_heads=[12, 16, 32, 48, 72])
        _sweep(common, opts, seq_len=[256, 512, 1024, 2048, 4096, 8192])
    _sweep(common, opts, per_head_dim=[16, 32, 64, 128])
    _sweep(common, opts, bs=[1], num_heads=[4], seq_len=[8192, 16384, 32768], sw_sz=[1024, 4096])


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--quick", action="store_true", help="a subset of every sweep")
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--graph", action="store_true", help="time graph replays instead of plain calls")
    args = ap.parse_args()
    opts = dict(warmup=args.warmup, iters=args.iters, graph=args.graph)
    benchmark_decode(opts, args.quick)
    benchmark_prefill(opts, use_bwd=False, quick=args.quick)
    benchmark_prefill(opts, use_bwd=True, quick=args.quick)


if __name__ == "__main__":
    main()
