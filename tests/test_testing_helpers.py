"""`triton_amd.testing`: the flop formulas (CPU) and the do_bench protocol (GPU)."""
import pytest

from triton_amd import testing


def test_flop_formulas_match_the_reference_expressions():
    # 03:437: perf = 2*M*N*K*1e-12/(ms*1e-3)
    assert testing.matmul_tflops(8192, 8192, 8192, 1.0) == pytest.approx(2 * 8192 ** 3 * 1e-12 / 1e-3)
    # 06:630-636: flops_per_matmul = 2*B*H*N*N*D, total = 2x, causal 0.5x, bwd 2.5x
    Z, H, N, D = 4, 32, 4096, 128
    per = 2.0 * Z * H * N * N * D
    assert testing.attention_tflops(Z, H, N, D, 1.0, False) == pytest.approx(2 * per * 1e-9)
    assert testing.attention_tflops(Z, H, N, D, 1.0, True) == pytest.approx(per * 1e-9)
    assert testing.attention_tflops(Z, H, N, D, 2.0, True, "bwd") == pytest.approx(2.5 * per * 1e-9 / 2)


def test_do_bench_rejects_unknown_return_mode():
    with pytest.raises(AssertionError):
        testing.do_bench(lambda: None, return_mode="mode")


@pytest.mark.gpu
def test_do_bench_times_a_gemm_and_orders_quantiles(gpu):
    import torch

    import triton_amd

    a = torch.randn(2048, 2048, device=gpu, dtype=torch.bfloat16)
    b = torch.randn(2048, 2048, device=gpu, dtype=torch.bfloat16)
    q = testing.do_bench(lambda: triton_amd.matmul(a, b), warmup=5, rep=20, quantiles=[0.5, 0.2, 0.8])
    assert len(q) == 3 and 0 < q[1] <= q[0] <= q[2]
    mean = testing.do_bench(lambda: triton_amd.matmul(a, b), warmup=5, rep=20)
    lo = testing.do_bench(lambda: triton_amd.matmul(a, b), warmup=5, rep=20, return_mode="min")
    assert 0 < lo <= mean * 1.5
    # a 2048^3 bf16 GEMM on this GPU is far below a millisecond
    assert q[0] < 1.0


def _sweep(calls):
    configs = [testing.Benchmark(x_names=["M", "N", "K"], x_vals=[128 * i for i in range(2, 5)], line_arg="provider",
                                 line_vals=["rocblas", "triton"], line_names=["rocBLAS", "Triton"],
                                 styles=[("green", "-"), ("blue", "-")], ylabel="TFLOPS", plot_name="matmul-performance-fp16",
                                 args={"fp8_inputs": False})]

    @testing.perf_report(configs)
    def benchmark(M, N, K, provider, fp8_inputs, do_bench):
        calls.append((M, N, K, provider, fp8_inputs))
        ms, lo, hi = do_bench(provider, M)
        perf = lambda t: 2 * M * N * K * 1e-12 / (t * 1e-3)
        return perf(ms), perf(hi), perf(lo)

    return benchmark


def test_perf_report_sweeps_x_values_and_lines_like_the_tutorial_benchmark(tmp_path, capsys):
    # the benchmark section of 03:405-441 with an injected timer: 1 ms per 256 rows for one line, half for the other
    calls = []
    bench = _sweep(calls)
    fake = lambda provider, M: tuple(f * M / 256 * (1.0 if provider == "rocblas" else 0.5) for f in (1.0, 0.9, 1.1))
    tables = bench.run(show_plots=True, print_data=True, save_path=str(tmp_path), return_df=True, do_bench=fake)
    assert calls == [(m, m, m, p, False) for m in (256, 384, 512) for p in ("rocblas", "triton")]
    t = tables[0]
    assert t.columns == ["M", "N", "K", "rocBLAS", "Triton"] and t.column("M") == [256, 384, 512]
    for m, slow, fast in zip(t.column("M"), t.column("rocBLAS"), t.column("Triton")):
        assert slow == pytest.approx(2 * m ** 3 * 1e-12 / (m / 256 * 1e-3)) and fast == pytest.approx(2 * slow)
    assert t.low[0][0] < t.rows[0][3] < t.high[0][0]      # (perf(max_ms), perf(min_ms)) bracket the median
    out = capsys.readouterr().out
    assert out.startswith("matmul-performance-fp16:\n") and "rocBLAS" in out and len(out.splitlines()) == 5
    lines = (tmp_path / "matmul-performance-fp16.csv").read_text().splitlines()
    assert lines[0] == "M,N,K,rocBLAS,Triton" and len(lines) == 4
    assert [float(x) for x in lines[1].split(",")] == pytest.approx([256, 256, 256, t.rows[0][3], t.rows[0][4]], abs=1e-6)   # written with save_precision = 6 digits
    assert t.to_pandas().shape == (3, 5)


def test_perf_report_single_benchmark_scalar_returns_and_diff_column():
    # the attention benchmark of 06:567-641 returns one number per call; one Benchmark (not a list) returns one table
    b = testing.Benchmark(x_names=["N_CTX"], x_vals=[2 ** i for i in range(10, 13)], line_arg="provider", line_vals=["a"],
                          line_names=["A"], plot_name="p", args={"H": 2})
    t = testing.perf_report(b)(lambda N_CTX, provider, H: N_CTX * H).run(return_df=True, diff_col=True)
    assert t.columns == ["N_CTX", "A", "Diff"] and t.rows == [[1024, 2048, 1024], [2048, 4096, 2048], [4096, 8192, 4096]]
    assert t.low == [[None]] * 3
    assert testing.perf_report(b)(lambda N_CTX, provider, H: 0).run() is None


def test_perf_report_rejects_x_tuples_of_the_wrong_length():
    b = testing.Benchmark(x_names=["M", "N"], x_vals=[(1, 2, 3)], line_arg="p", line_vals=["a"], line_names=["A"], plot_name="p", args={})
    with pytest.raises(ValueError, match="Expected 2 values"):
        testing.perf_report(b)(lambda M, N, p: 0).run()
    with pytest.raises(ValueError):
        testing.Benchmark(x_names=["M"], x_vals=[1], line_arg="p", line_vals=["a", "b"], line_names=["A"], plot_name="p", args={})


@pytest.mark.gpu
def test_tutorial_benchmark_sections_run_against_this_package(gpu, tmp_path):
    """The benchmark sections of 03:405-441 and 06:567-641 with `triton.testing` -> `triton_amd.testing` and the
    operators from `triton_amd`, on two x values each."""
    import torch

    import triton_amd

    mm = testing.Benchmark(x_names=["M", "N", "K"], x_vals=[128 * i for i in (8, 16)], line_arg="provider", line_vals=["rocblas", "triton"],
                           line_names=["rocBLAS", "Triton"], styles=[("green", "-"), ("blue", "-")], ylabel="TFLOPS",
                           plot_name="matmul-performance-fp16", args={"fp8_inputs": False})

    @testing.perf_report([mm])
    def benchmark(M, N, K, provider, fp8_inputs):
        a = torch.randn((M, K), device="cuda", dtype=torch.float16)
        b = torch.randn((K, N), device="cuda", dtype=torch.float16)
        quantiles = [0.5, 0.2, 0.8]
        if provider == "rocblas":
            ms, min_ms, max_ms = testing.do_bench(lambda: torch.matmul(a, b), warmup=5, rep=20, quantiles=quantiles)
        if provider == "triton":
            ms, min_ms, max_ms = testing.do_bench(lambda: triton_amd.matmul(a, b), warmup=5, rep=20, quantiles=quantiles)
        perf = lambda ms: 2 * M * N * K * 1e-12 / (ms * 1e-3)
        return perf(ms), perf(max_ms), perf(min_ms)

    t = benchmark.run(show_plots=True, print_data=True, save_path=str(tmp_path), return_df=True)[0]
    assert t.column("M") == [1024, 2048] and all(v > 10 for v in t.column("Triton"))   # TFLOP/s
    assert (tmp_path / "matmul-performance-fp16.csv").exists()

    fa = testing.Benchmark(x_names=["N_CTX"], x_vals=[1024, 2048], line_arg="provider", line_vals=["triton-fp16"], line_names=["Triton [FP16]"],
                           styles=[("red", "-")], ylabel="ms", plot_name="fused-attention-fwd",
                           args={"H": 4, "BATCH": 2, "HEAD_DIM": 64, "mode": "bwd", "causal": True})

    @testing.perf_report(fa)
    def bench_flash_attention(BATCH, H, N_CTX, HEAD_DIM, causal, mode, provider, device="cuda"):
        q, k, v = (torch.randn((BATCH, H, N_CTX, HEAD_DIM), dtype=torch.float16, device=device, requires_grad=True) for _ in range(3))
        fn = lambda: triton_amd.attention(q, k, v, causal, 1.3)
        o = fn()
        do = torch.randn_like(o)
        fn = lambda: o.backward(do, retain_graph=True)
        ms = testing.do_bench(fn, warmup=5, rep=20)
        return testing.attention_tflops(BATCH, H, N_CTX, HEAD_DIM, ms, causal, mode)

    t = bench_flash_attention.run(save_path=str(tmp_path), print_data=True, return_df=True)
    assert t.column("N_CTX") == [1024, 2048] and all(v > 1 for v in t.column("Triton [FP16]"))
    assert testing.get_max_tensorcore_tflops(torch.bfloat16, 2400000) == pytest.approx(2500, rel=0.02)
