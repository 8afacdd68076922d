"""Timing helper with the protocol of the reference's `triton.testing.do_bench`
(python/triton/testing.py:84-160): one warm call, an estimate from five flushed runs, then
`warmup` / `rep` milliseconds worth of calls, every timed call preceded by a write over a buffer
larger than the last-level cache and bracketed by its own pair of device events.

`do_bench` keeps the reference's signature, defaults and return conventions; `do_bench_cudagraph`
(python/triton/testing.py:19-82) is the same measurement from inside a captured HIP graph.  The flush buffer is 512 MB here:
MI355X's memory-side cache holds 256 MB, the size the reference clears.

`Benchmark`, `perf_report` and `Mark.run` (python/triton/testing.py:214-388) are the sweep harness that the
tutorials' benchmark sections are written in (`03:405-441`, `06:567-641`): with `triton.testing` replaced by
this module and `matmul` / `attention` taken from `triton_amd`, those sections run as they stand.  The tables
are printed and written as CSV with the standard library; nothing is plotted (`show_plots` is accepted and
ignored, `styles`, `x_log`, `y_log`, `xlabel`, `ylabel` are kept as attributes only).
`get_max_tensorcore_tflops` (python/triton/testing.py:404-426) becomes the dense MFMA rate of the device:
CUs x 4 SIMDs x flop per SIMD and cycle x clock.
"""
from __future__ import annotations

import csv
import os

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


def do_bench_cudagraph(fn, rep=20, grad_to_none=None, return_mode="mean"):
    """`do_bench` without host overhead between the calls (python/triton/testing.py:19-82, same signature and protocol):
    `fn` is captured into a HIP graph, first once for an estimate, then `rep` ms worth of calls unrolled in one graph,
    which is replayed ten times; the result is the time per call in ms over those replays (`return_mode`).  No cache
    flush between the calls.  Must run on a side stream, like the reference's (a capture on the default stream is
    refused); `fn` has been called once outside any capture before the first one, so first-call set-up never lands in
    a graph.  The operators of this package record kernels only (no runtime allocation or memset inside the library)."""
    assert return_mode in _RETURN_MODES
    import torch

    if torch.cuda.current_stream() == torch.cuda.default_stream():
        raise RuntimeError("Cannot capture graph in default stream. Please use side stream in benchmark code.")

    def reset_grads():
        if grad_to_none is not None:
            for x in grad_to_none:
                x.grad = None

    def capture(calls):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(calls):
                reset_grads()
                fn()
        torch.cuda.synchronize()
        return graph

    def replay_ms(graph):
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        graph.replay()
        end.record()
        torch.cuda.synchronize()
        return begin.elapsed_time(end)

    fn()
    torch.cuda.synchronize()
    if grad_to_none is not None:
        for x in grad_to_none:
            x.detach_()
            x.requires_grad_(True)
            x.grad = None
    estimate_ms = replay_ms(capture(1))
    n_repeat = max(1, int(rep / estimate_ms))
    graph = capture(n_repeat)
    times = torch.tensor([replay_ms(graph) / n_repeat for _ in range(10)], dtype=torch.float)
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


class Benchmark:
    """One sweep: the benchmarked function is called once per x value and per line value.  Constructor
    arguments as python/triton/testing.py:219-273: `x_names` are the swept argument names and `x_vals` their
    values (a scalar is given to every x name, a tuple / list supplies one value per name), `line_arg` is the
    argument that tells the lines (providers) apart with values `line_vals` and column titles `line_names`,
    `plot_name` names the table and its CSV file, `args` are fixed keyword arguments."""

    def __init__(self, x_names, x_vals, line_arg, line_vals, line_names, plot_name, args,
                 xlabel="", ylabel="", x_log=False, y_log=False, styles=None):
        self.x_names, self.x_vals = list(x_names), list(x_vals)
        self.line_arg, self.line_vals, self.line_names = line_arg, list(line_vals), list(line_names)
        self.plot_name, self.args = plot_name, dict(args)
        self.xlabel, self.ylabel, self.x_log, self.y_log, self.styles = xlabel, ylabel, x_log, y_log, styles
        if len(self.line_vals) != len(self.line_names):
            raise ValueError(f"{len(self.line_vals)} line values for {len(self.line_names)} line names")


class ResultTable:
    """The outcome of one Benchmark: column titles and rows of numbers (what the reference keeps in a pandas
    frame, python/triton/testing.py:287-354).  `low` / `high` hold the second and third value of every
    measurement that returned a triple (None otherwise); they are not printed, as in the reference."""

    def __init__(self, name, columns):
        self.name, self.columns = name, list(columns)
        self.rows, self.low, self.high = [], [], []

    def add_diff(self):
        self.columns.append("Diff")
        self.rows = [row + [row[-1] - row[-2]] for row in self.rows]

    @staticmethod
    def _cell(v, precision):
        if isinstance(v, float):
            return f"{v:.{precision}f}"
        return "" if v is None else str(v)

    def to_string(self, precision=6):
        cells = [["", *self.columns]] + [[str(i), *(self._cell(v, precision) for v in row)] for i, row in enumerate(self.rows)]
        width = [max(len(r[c]) for r in cells) for c in range(len(cells[0]))]
        return "\n".join("  ".join(x.rjust(w) for x, w in zip(r, width)) for r in cells)

    def to_csv(self, path, precision=6):
        with open(path, "w", newline="") as f:
            w = csv.writer(f)
            w.writerow(self.columns)
            for row in self.rows:
                w.writerow([self._cell(v, precision) for v in row])

    def column(self, title):
        i = self.columns.index(title)
        return [row[i] for row in self.rows]

    def to_pandas(self):
        import pandas

        return pandas.DataFrame(self.rows, columns=self.columns)


class Mark:
    """A function bound to its sweeps; `run` executes them (python/triton/testing.py:276-388)."""

    def __init__(self, fn, benchmarks):
        self.fn, self.benchmarks = fn, benchmarks

    def __call__(self, *args, **kwargs):
        return self.fn(*args, **kwargs)

    def _run(self, bench, save_path, print_data, diff_col=False, save_precision=6, **kwargs):
        table = ResultTable(bench.plot_name, bench.x_names + bench.line_names)
        for x in bench.x_vals:
            xs = list(x) if isinstance(x, (list, tuple)) else [x] * len(bench.x_names)
            if len(xs) != len(bench.x_names):
                raise ValueError(f"Expected {len(bench.x_names)} values, got {x}")
            mid, low, high = [], [], []
            for line in bench.line_vals:
                ret = self.fn(**dict(zip(bench.x_names, xs)), **{bench.line_arg: line}, **bench.args, **kwargs)
                try:
                    m, lo, hi = ret
                except TypeError:
                    m, lo, hi = ret, None, None
                mid.append(m), low.append(lo), high.append(hi)
            table.rows.append(xs + mid), table.low.append(low), table.high.append(high)
        if diff_col and len(table.columns) == 2:
            table.add_diff()
        if print_data:
            print(f"{bench.plot_name}:")
            print(table.to_string(save_precision))
        if save_path:
            table.to_csv(os.path.join(save_path, f"{bench.plot_name}.csv"), save_precision)
        return table

    def run(self, show_plots=False, print_data=False, save_path="", return_df=False, **kwargs):
        """Runs every sweep.  `return_df=True` returns the tables (one, or a list when a list of Benchmarks
        was given) - `ResultTable` objects; `.to_pandas()` turns one into the frame the reference returns."""
        single = isinstance(self.benchmarks, Benchmark)
        if save_path:
            os.makedirs(save_path, exist_ok=True)
        tables = [self._run(b, save_path, print_data, **kwargs) for b in ([self.benchmarks] if single else self.benchmarks)]
        if return_df:
            return tables[0] if single else tables
        return None


def perf_report(benchmarks):
    """Decorator: `@perf_report(configs)` turns a function into a `Mark` whose `.run()` sweeps it."""
    return lambda fn: Mark(fn, benchmarks)


# dense MFMA flop per compute unit and cycle on gfx950 (a 16x16x32 16-bit MFMA is 16384 flop in 16 cycles on each
# of a CU's four SIMDs; 256 CUs x 2.4 GHz x 4096 = 2.5 PFLOP/s, the published peak)
_MFMA_FLOP_PER_CU_CYCLE = {"fp32": 256, "16bit": 4096, "8bit": 8192, "4bit": 16384}


def get_max_tensorcore_tflops(dtype, clock_rate, device=None):
    """Dense matrix-core peak in TFLOP/s at `clock_rate` (kHz, as the reference passes it): compute units x
    flop per CU and cycle x clock.  16-bit types 4096 flop per CU and cycle (256 CUs at 2.4 GHz: 2.5 PFLOP/s),
    8-bit types twice that, fp32 256; `dtype` may be a torch dtype or one of "mxfp4", "mxfp8"."""
    import torch

    if device is None:
        device = torch.cuda.current_device()
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    name = str(dtype).replace("torch.", "")
    if name in ("float16", "bfloat16", "int16"):
        per = _MFMA_FLOP_PER_CU_CYCLE["16bit"]
    elif name.startswith("float8") or name in ("int8", "mxfp8"):
        per = _MFMA_FLOP_PER_CU_CYCLE["8bit"]
    elif name in ("mxfp4", "float4_e2m1fn_x2"):
        per = _MFMA_FLOP_PER_CU_CYCLE["4bit"]
    elif name in ("float32", "int32"):
        per = _MFMA_FLOP_PER_CU_CYCLE["fp32"]
    else:
        raise RuntimeError("dtype not supported")
    return cus * clock_rate * per * 1e-9
