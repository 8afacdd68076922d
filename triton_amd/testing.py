"""Timing helper with the protocol of the reference's `triton.testing.do_bench`
(python/triton/testing.py:84-160): one warm call, an estimate from five flushed runs, then
`warmup` / `rep` milliseconds worth of calls, every timed call preceded by a write over a buffer
larger than the last-level cache and bracketed by its own pair of device events.

Same signature, defaults and return conventions as the reference, so its benchmark scripts
(`03:424-441`, `06:599-641`) run unchanged against this module.  The flush buffer is 512 MB here:
MI355X's memory-side cache holds 256 MB, the size the reference clears.
"""
from __future__ import annotations

_RETURN_MODES = ("min", "max", "mean", "median")
_FLUSH_BYTES = 512 * 1024 * 1024


def do_bench(fn, warmup=25, rep=100, grad_to_none=None, quantiles=None, fast_flush=True, return_mode="mean"):
    """Run `fn` repeatedly on the current device and return its runtime in milliseconds.

    warmup, rep     time budgets in ms for the untimed and the timed calls
    grad_to_none    tensors whose `.grad` is reset before every timed call (backward benchmarks)
    quantiles       if given, return these quantiles of the per-call times instead of `return_mode`
    fast_flush      flush with a 4-byte-element fill (fewer, wider stores) instead of a byte fill
    return_mode     "min" | "max" | "mean" | "median"
    """
    assert return_mode in _RETURN_MODES
    import torch

    fn()
    torch.cuda.synchronize()

    if fast_flush:
        flush = torch.empty(_FLUSH_BYTES // 4, dtype=torch.int32, device="cuda")
    else:
        flush = torch.empty(_FLUSH_BYTES, dtype=torch.int8, device="cuda")

    first, second = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    first.record()
    for _ in range(5):
        flush.zero_()
        fn()
    second.record()
    torch.cuda.synchronize()
    estimate_ms = first.elapsed_time(second) / 5

    n_warmup = max(1, int(warmup / estimate_ms))
    n_repeat = max(1, int(rep / estimate_ms))
    begins = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for _ in range(n_warmup):
        fn()
    for i in range(n_repeat):
        if grad_to_none is not None:
            for x in grad_to_none:
                x.grad = None
        flush.zero_()
        begins[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    times = torch.tensor([b.elapsed_time(e) for b, e in zip(begins, ends)], dtype=torch.float)
    if quantiles is not None:
        out = torch.quantile(times, torch.tensor(quantiles, dtype=torch.float)).tolist()
        return out[0] if len(out) == 1 else out
    return getattr(torch, return_mode)(times).item()


def matmul_tflops(M: int, N: int, K: int, ms: float) -> float:
    """`2*M*N*K` flop over `ms` milliseconds, the figure of merit of tutorial 03 (`03:437`)."""
    return 2.0 * M * N * K * 1e-12 / (ms * 1e-3)


def attention_tflops(Z: int, H: int, N_CTX: int, D: int, ms: float, causal: bool, mode: str = "fwd") -> float:
    """The reference's attention flop count (`06:630-636`): two matmuls of `2*Z*H*N^2*D` forward,
    halved when causal, 2.5x that for the backward (2.0 backward + 0.5 recompute)."""
    assert mode in ("fwd", "bwd")
    total = 2 * (2.0 * Z * H * N_CTX * N_CTX * D)
    if causal:
        total *= 0.5
    if mode == "bwd":
        total *= 2.5
    return total * 1e-12 / (ms * 1e-3)
