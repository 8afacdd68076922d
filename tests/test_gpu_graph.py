"""GPU: the operators under HIP graph capture.  The reference's kernels are launched from captured graphs as a matter of
course (python/triton/testing.py:19-82, `do_bench_cudagraph`, captures the benchmarked call); here a call is a C-ABI
entry point that launches on the stream it is given and neither allocates nor clears memory through the runtime, so a
capture records kernels only.  The test captures one of everything - tile GEMM, the split-K route of `matmul` (its
workspace comes from torch's allocator, i.e. the graph's private pool), block-scaled GEMM, the stream-K entry point with
the static scratch array, attention forward and backward through autograd - and replays the graph several times on new
input values, with the program's own eager launches and synchronisations between the replays; every replay must give
the bits of the eager call on the same inputs (same kernels, fixed summation orders)."""
import pytest
import torch

import triton_amd
from triton_amd import _lib

pytestmark = pytest.mark.gpu


def _work(lib, t):
    c1 = triton_amd.matmul(t["a"], t["b"])                       # 2048 x 2048 x 1024: tile kernel
    c2 = triton_amd.matmul(t["a2"], t["b2"])                     # 256 x 384 x 8192: split over K, two launches
    c3 = triton_amd.mx_matmul(t["pa"], t["sa"], t["pb"], t["sb"], "mxfp4", out_dtype=torch.bfloat16)
    a, b, c4 = t["a"], t["b"], t["c4"]                           # 64 tiles of 256 x 256 over one program per CU
    rc = lib.mi355_gemm_streamk_static(a.data_ptr(), b.data_ptr(), c4.data_ptr(), a.shape[0], b.shape[1], a.shape[1],
                                       a.stride(0), a.stride(1), b.stride(0), b.stride(1), c4.stride(0), c4.stride(1),
                                       _lib.BF16, _lib.BF16, None, None, _lib.ACT_NONE, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    o = triton_amd.attention(t["q"], t["k"], t["v"], True, 0.125)
    dq, dk, dv = torch.autograd.grad(o, (t["q"], t["k"], t["v"]), t["do"])
    return [c1, c2, c3, c4, o.detach(), dq, dk, dv]


def test_captured_graph_replays_give_the_bits_of_the_eager_calls(gpu):
    lib = _lib.load()
    g = torch.Generator(device="cpu").manual_seed(3)
    bf = lambda *s: torch.randn(*s, generator=g).bfloat16().to(gpu)
    u8 = lambda lo, hi, *s: torch.randint(lo, hi, s, generator=g, dtype=torch.uint8).to(gpu)
    t = {"a": bf(2048, 1024), "b": bf(1024, 2048), "a2": bf(256, 8192), "b2": bf(8192, 384),
         "pa": u8(0, 256, 512, 512), "sa": u8(123, 132, 512, 32), "pb": u8(0, 256, 256, 512), "sb": u8(123, 132, 256, 32),
         "c4": torch.empty(2048, 2048, dtype=torch.bfloat16, device=gpu),
         "q": (bf(2, 4, 512, 64) * 0.5).requires_grad_(), "k": (bf(2, 4, 512, 64) * 0.5).requires_grad_(),
         "v": (bf(2, 4, 512, 64) * 0.5).requires_grad_(), "do": bf(2, 4, 512, 64)}
    # first calls outside the capture, on a side stream as torch asks: kernel attributes, the per-device address of
    # the scratch array and the library's cached device facts are set up by then
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            _work(lib, t)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = _work(lib, t)
    torch.cuda.synchronize()

    names = ["matmul", "matmul (split-K)", "mx_matmul", "stream-K static", "attention o", "dq", "dk", "dv"]
    for replay in range(4):
        # new values in the captured tensors (eager kernels), the eager results on them, then the replay
        with torch.no_grad():
            for key in ("a", "b", "a2", "b2", "q", "k", "v", "do"):
                t[key].copy_(torch.randn(t[key].shape, generator=g).bfloat16() * (0.5 if key in "qkv" else 1.0))
            t["pa"].copy_(u8(0, 256, 512, 512))
            t["sb"].copy_(u8(123, 132, 256, 32))
        ref_c4 = torch.empty_like(t["c4"])
        saved, t["c4"] = t["c4"], ref_c4
        want = [w.clone() for w in _work(lib, t)]
        t["c4"] = saved
        for o in outs:
            o.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, ref in zip(names, outs, want):
            assert torch.equal(got, ref), (replay, name)


def test_do_bench_cudagraph_times_a_captured_call(gpu):
    # the reference's graph-based timer (python/triton/testing.py:19-82): refuses the default stream, and on a side
    # stream agrees with the per-call events of do_bench on a kernel long enough for neither to be launch bound
    from triton_amd.testing import do_bench, do_bench_cudagraph
    a = torch.randn(4096, 4096, device=gpu, dtype=torch.bfloat16)
    b = torch.randn(4096, 4096, device=gpu, dtype=torch.bfloat16)
    fn = lambda: triton_amd.matmul(a, b)
    with pytest.raises(RuntimeError, match="side stream"):
        do_bench_cudagraph(fn)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ms_graph = do_bench_cudagraph(fn, rep=20)
    torch.cuda.current_stream().wait_stream(side)
    ms_events = do_bench(fn, warmup=5, rep=20, return_mode="median")
    print(f"4096^3 bf16: {ms_graph:.4f} ms per call inside a graph, {ms_events:.4f} ms flushed with events")
    assert 0.05 < ms_graph < 1.0 and 0.3 < ms_graph / ms_events < 2.0
