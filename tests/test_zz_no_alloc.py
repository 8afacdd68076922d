"""GPU: the entry point that allocates nothing (mi355_gemm_streamk_static: stream-K with the partial-tile
workspace in the library's static device array) against the existing entry point it is a variant of
(mi355_gemm_streamk with a caller's workspace), through the C ABI.  Same kernels, same order of the
partial sums, so the outputs must agree bit for bit - on two calls in a row, the second on a smaller
input (the array keeps the first call's contents), and while no device memory is allocated."""
import numpy as np
import pytest
import torch

from triton_amd import _lib
from util import set_knob

pytestmark = pytest.mark.gpu


def _call(lib, which, a, b, c, ws=None):
    M, K = a.shape
    N = b.shape[1]
    args = [a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K,
            a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
            _lib.BF16, _lib.BF16, None, None, _lib.ACT_NONE]
    stream = torch.cuda.current_stream().cuda_stream
    if which == "static":
        return lib.mi355_gemm_streamk_static(*args, stream)
    return lib.mi355_gemm_streamk(*args, ws.data_ptr(), ws.numel(), stream)


@pytest.mark.parametrize("nprog", [None, 7])
def test_static_scratch_stream_k_matches_workspace_stream_k(gpu, monkeypatch, nprog):
    # nprog None: one program per CU - more programs than tiles here, i.e. split-K, every tile summed from
    # several partial slots; 7: ranges that begin and end inside tiles
    if nprog is not None:
        set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", nprog)
    lib = _lib.load()
    ws = torch.empty(lib.mi355_query(_lib.Q_STREAMK_WORKSPACE_BYTES), device=gpu, dtype=torch.uint8)
    g = torch.Generator(device="cpu").manual_seed(7)
    shapes = [(1024, 768, 4096), (512, 256, 1024)]          # the second call is the smaller input
    tensors = []
    for (M, N, K) in shapes:
        a = torch.randn(M, K, generator=g).bfloat16().to(gpu)
        b = torch.randn(K, N, generator=g).bfloat16().to(gpu)
        tensors.append((a, b, torch.empty(M, N, device=gpu, dtype=torch.bfloat16),
                        torch.empty(M, N, device=gpu, dtype=torch.bfloat16)))
    # the reference results first (caller's workspace), then the static calls back to back with the
    # allocator watched: nothing may be allocated or freed between the two counters
    for (a, b, want, _) in tensors:
        assert _call(lib, "workspace", a, b, want, ws) == 0
    assert _call(lib, "static", *tensors[0][:2], tensors[0][3]) == 0     # (first call on the device: address look-up)
    torch.cuda.synchronize()
    for t in tensors:
        t[3].zero_()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    stats_before = torch.cuda.memory_stats().get("num_alloc_retries", 0), torch.cuda.memory_allocated()
    for (a, b, _, got) in tensors:
        assert _call(lib, "static", a, b, got) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, "device memory in use changed across the calls"
    assert stats_before == (torch.cuda.memory_stats().get("num_alloc_retries", 0), torch.cuda.memory_allocated())
    for (a, b, want, got), shape in zip(tensors, shapes):
        assert torch.equal(got, want), shape
        ref = a[:8].double().cpu().numpy() @ b.double().cpu().numpy()
        assert np.allclose(got[:8].float().cpu().numpy(), ref, rtol=1e-2, atol=1e-2)


def test_static_scratch_rejects_bad_arguments(gpu):
    lib = _lib.load()
    assert lib.mi355_gemm_streamk_static(None, None, None, 256, 256, 256, 256, 1, 256, 1, 256, 1,
                                         _lib.BF16, _lib.BF16, None, None, 0, None) == -1
    assert b"scratch" in lib.mi355_strerror(-6)
