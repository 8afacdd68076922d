"""Launch-path behaviour that the reference tests in python/test/unit/runtime/test_launch.py:
hooks that see the launch record (:18-43), no growth of the Python heap over repeated launches
(:46-69), and the per-launch host time against its 46 us budget (:74-76, disabled there).  Plus the
stream contract of the reference launcher: work goes to torch's current stream (python/triton/runtime/jit.py:588-589)."""
import gc
import time
import tracemalloc

import numpy as np
import pytest
import torch

import triton_amd
from triton_amd import _lib, hooks

pytestmark = pytest.mark.gpu


def test_hooks_see_the_launch_record(gpu):
    seen = []

    def enter(md):
        seen.append(("enter", md.get()))

    def leave(md):
        seen.append(("exit", md.get()))

    a = torch.randn(256, 128, device=gpu, dtype=torch.float16)
    b = torch.randn(128, 512, device=gpu, dtype=torch.float16)
    hooks.Launch.launch_enter_hook, hooks.Launch.launch_exit_hook = enter, leave
    try:
        triton_amd.matmul(a, b)
        q = torch.randn(1, 2, 128, 64, device=gpu, dtype=torch.float16)
        triton_amd.attention(q, q, q, True, 0.125)
    finally:
        hooks.Launch.launch_enter_hook = hooks.Launch.launch_exit_hook = None
    assert [s[0] for s in seen] == ["enter", "exit", "enter", "exit"]
    rec = seen[0][1]
    assert rec["name"] == "mi355_gemm [M=256, N=512, K=128]"          # 09:37
    assert rec["flops16"] == 2.0 * 256 * 512 * 128 and "flops8" not in rec
    assert rec["bytes"] == 2 * (256 * 128 + 512 * 128)                # 09:43
    assert rec["stream"] == torch.cuda.current_stream().cuda_stream
    rec = seen[2][1]
    assert rec["flops16"] == 4.0 * 1 * 2 * 128 * 128 * 64 * 0.5      # 06:630-634
    # without hooks nothing is recorded
    triton_amd.matmul(a, b)
    assert len(seen) == 4


def test_fp8_record_counts_flops8(gpu):
    seen = []
    a = torch.randn(64, 64, device=gpu).to(torch.float8_e4m3fn)
    b = torch.randn(64, 64, device=gpu).to(torch.float8_e4m3fn).T
    hooks.Launch.launch_enter_hook = lambda md: seen.append(md.get())
    try:
        triton_amd.matmul_like_input(a, b)
    finally:
        hooks.Launch.launch_enter_hook = None
    assert seen[0]["flops8"] == 2.0 * 64 ** 3 and seen[0]["bytes"] == 2 * 64 * 64


def test_memory_leak(gpu):
    # the reference's test, with matmul as the kernel: 100 launches may not grow the heap by 30 kB
    a = torch.randn(64, 64, device=gpu, dtype=torch.float16)
    b = torch.randn(64, 64, device=gpu, dtype=torch.float16)
    q = torch.randn(1, 1, 128, 64, device=gpu, dtype=torch.float16)
    tracemalloc.start()
    try:
        triton_amd.matmul(a, b)
        triton_amd.attention(q, q, q, False, 0.125)
        gc.collect()
        begin, _ = tracemalloc.get_traced_memory()
        for _ in range(100):
            triton_amd.matmul(a, b)
            triton_amd.attention(q, q, q, False, 0.125)
        gc.collect()
        end, _ = tracemalloc.get_traced_memory()
        assert end - begin < 30000
    finally:
        tracemalloc.stop()


def test_launch_goes_to_the_current_stream_and_is_ordered_on_it(gpu):
    # A producer kernel on a side stream, then matmul on the same stream without any host sync: the
    # product must see the produced operand.  The default stream stays idle throughout.
    side = torch.cuda.Stream(device=gpu)
    a = torch.zeros(1024, 1024, device=gpu, dtype=torch.float16)
    b = torch.eye(1024, device=gpu, dtype=torch.float16)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        for _ in range(20):               # keep the stream busy so that an unordered launch would run early
            a.add_(1.0)
        c = triton_amd.matmul(a, b)
    side.synchronize()
    assert torch.equal(c, torch.full_like(c, 20.0))


def test_host_time_per_launch(gpu):
    # Host cost of one call of the wrapper (argument checks, output allocation, the C-ABI call), with
    # the GPU kept idle enough not to block: the reference's budget for a launch is 46 us.
    a = torch.randn(16, 64, device=gpu, dtype=torch.float16)
    b = torch.randn(64, 64, device=gpu, dtype=torch.float16)
    for _ in range(50):
        triton_amd.matmul(a, b)
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(5):
        t0 = time.perf_counter()
        for _ in range(200):
            triton_amd.matmul(a, b)
        best = min(best, (time.perf_counter() - t0) / 200)
        torch.cuda.synchronize()
    print(f"host time per matmul() call: {best * 1e6:.1f} us")
    assert best < 46e-6


def test_torch_extension_is_the_default_binding_and_agrees_with_ctypes(gpu, monkeypatch):
    # The PyTorch-ROCm extension (tensor objects in, c10::hip::getCurrentHIPStream(), one C-ABI call) is what the
    # operators use when it is built; ctypes is the same C ABI reached from Python.  Same kernels, same bits;
    # and the host time per call of both bindings, for the record.
    from triton_amd import _lib

    assert _lib.ext() is not None, "the torch extension was not built (python -m triton_amd.build)"
    a = torch.randn(256, 512, device=gpu, dtype=torch.bfloat16)
    b = torch.randn(512, 384, device=gpu, dtype=torch.bfloat16)
    bias = torch.randn(1, 384, device=gpu, dtype=torch.float32)
    q, k, v = (torch.randn(1, 2, 256, 64, device=gpu, dtype=torch.float16).requires_grad_() for _ in range(3))
    do = torch.randn(1, 2, 256, 64, device=gpu, dtype=torch.float16)

    def run():
        c = triton_amd.matmul(a, b, activation="leaky_relu", add=bias)
        o = triton_amd.attention(q, k, v, True, 0.125)
        grads = torch.autograd.grad(o, (q, k, v), do)
        return (c, o.detach(), *grads)

    def host_us():
        x = torch.randn(16, 64, device=gpu, dtype=torch.float16)
        y = torch.randn(64, 64, device=gpu, dtype=torch.float16)
        for _ in range(50):
            triton_amd.matmul(x, y)
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(5):
            t0 = time.perf_counter()
            for _ in range(200):
                triton_amd.matmul(x, y)
            best = min(best, (time.perf_counter() - t0) / 200)
            torch.cuda.synchronize()
        return best * 1e6

    with_ext = run()
    us_ext = host_us()
    monkeypatch.setattr(_lib, "_ext", None)          # ctypes from here on
    with_ctypes = run()
    us_ctypes = host_us()
    for x, y in zip(with_ext, with_ctypes):
        assert torch.equal(x, y)
    print(f"host time per matmul() call: torch extension {us_ext:.1f} us, ctypes {us_ctypes:.1f} us")
    with torch.cuda.stream(torch.cuda.Stream(device=gpu)):
        monkeypatch.setattr(_lib, "_ext", False)     # (re-resolved: the extension again) on a side stream
        e = torch.eye(512, device=gpu, dtype=torch.bfloat16)
        acc = torch.zeros(512, 512, device=gpu, dtype=torch.bfloat16)
        for _ in range(10):
            acc.add_(1.0)
        out = triton_amd.matmul(acc, e)
    torch.cuda.synchronize()
    assert torch.equal(out, torch.full_like(out, 10.0))   # launched on, and ordered by, the current (side) stream


@pytest.mark.gpu
def test_clock_and_mfma_burn_probes(gpu):
    """The two measurement entries: the clock probe reports a plausible shader clock next to a burn of every MFMA
    shape, a burn launch finishes and leaves its sink alone, and bad arguments are rejected before any launch."""
    lib = _lib.load()
    sink = torch.zeros(4, device=gpu, dtype=torch.float32)
    ticks = torch.zeros(2, device=gpu, dtype=torch.int64)
    stream = torch.cuda.current_stream().cuda_stream
    side = torch.cuda.Stream(device=gpu)
    for shape in range(8):
        for rnd in (0, 1):
            assert lib.mi355_mfma_burn(sink.data_ptr(), shape, rnd, 200, 1, stream) == 0
    assert lib.mi355_clock_probe(ticks.data_ptr(), 2000, side.cuda_stream) == 0   # 2 ms next to the queued burns
    torch.cuda.synchronize()
    assert torch.equal(sink.cpu(), torch.zeros(4))
    cyc, real = ticks.tolist()
    mhz = cyc / real * lib.mi355_query(_lib.Q_WALL_CLOCK_KHZ) / 1e3
    assert 90 < mhz < 2600, mhz
    for bad in ((0, 0, 0, 100, 1), (sink.data_ptr(), 8, 0, 100, 1), (sink.data_ptr(), 0, 0, 0, 1), (sink.data_ptr(), 0, 0, 100, 3)):
        assert lib.mi355_mfma_burn(*bad, stream) == -1


@pytest.mark.gpu
def test_power_probe_module_reports_every_leg(gpu, capsys):
    from triton_amd import power_probe

    assert power_probe.main(["--seconds", "0.05", "--json"]) == 0
    import json

    rec = json.loads(capsys.readouterr().out)
    assert len(rec["legs"]) == 16 and all(leg["tflops"] > 100 for leg in rec["legs"])
    # the constant-operand legs are never slower than the random ones by more than noise (less switching, same work)
    by = {(leg["shape"], leg["operands"]): leg["tflops"] for leg in rec["legs"]}
    assert by[("bf16 16x16x32", "constant")] > 0.9 * by[("bf16 16x16x32", "random")]
