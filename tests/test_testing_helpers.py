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
