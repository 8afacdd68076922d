"""GPU parity: grouped GEMM through the C ABI (`group_gemm_fn`) against the CPU oracle.
The reference's own check is `torch.allclose(ref, out, atol=1e-2, rtol=0)` on rand() inputs of
sizes 1024, 512, 256, 128 (python/tutorials/08-grouped-gemm.py:190-214)."""
import numpy as np
import pytest
import torch

import triton_amd
from oracle import formats, gemm
from util import bits_equal, from_np, to_np, set_knob

pytestmark = pytest.mark.gpu


def _run(gpu, ga, gb, dtype, **kw):
    ta = [from_np(a, dtype, gpu) for a in ga]
    tb = [from_np(b, dtype, gpu) for b in gb]
    return [to_np(c) for c in triton_amd.group_gemm_fn(ta, tb, **kw)]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_reference_example_sizes(gpu, dtype):
    # 08:190-205: square problems 1024, 512, 256, 128 of uniform [0, 1) values
    rng = np.random.default_rng(0)
    ga = [formats.round_to(rng.random((d, d)).astype(np.float32), dtype) for d in (1024, 512, 256, 128)]
    gb = [formats.round_to(rng.random((d, d)).astype(np.float32), dtype) for d in (1024, 512, 256, 128)]
    outs = _run(gpu, ga, gb, dtype)
    for a, b, c in zip(ga, gb, outs):
        ref = gemm.matmul_closed_form(a, b, out_dtype=dtype)
        # results reach 2^8: one unit in the last place is 0.25 (fp16) / 2 (bf16), so the reference's
        # absolute 1e-2 only holds where both sides round the same way; the bar here is rtol 1e-2
        assert np.allclose(c, ref, rtol=1e-2, atol=1e-2)
        assert np.mean(c == ref) > 0.98


@pytest.mark.parametrize("big_min", [None, 1])
@pytest.mark.parametrize("nprog", [0, 1, 7, 100])
def test_ragged_problems_are_bit_exact_on_integers(gpu, nprog, big_min, monkeypatch):
    # partial tiles, a single row, K tails (K % 32 != 0), and problems without 16-byte rows; once with
    # the tile size the library picks for this group (128x128: fewer 256x256 tiles than CUs) and once
    # with the 256x256 form forced (MI355_GROUPED_BIG_MIN=1)
    if big_min is not None:
        set_knob(monkeypatch, "MI355_GROUPED_BIG_MIN", str(big_min))
    rng = np.random.default_rng(nprog)
    shapes = [(256, 128, 64), (130, 72, 40), (1, 304, 8), (128, 128, 128), (100, 70, 50), (37, 19, 7), (300, 264, 520)]
    ga = [rng.integers(-2, 3, size=(m, k)).astype(np.float32) for m, n, k in shapes]
    gb = [rng.integers(-2, 3, size=(k, n)).astype(np.float32) for m, n, k in shapes]
    ref = gemm.grouped_matmul(ga, gb, num_programs=max(nprog, 1), out_dtype="fp32")
    for dtype in ("fp16", "bf16"):
        outs = _run(gpu, ga, gb, dtype, num_programs=nprog)
        for c, r in zip(outs, ref):
            assert bits_equal(c, r)   # integer results below 2^11 are exact in fp16 and bf16


def test_strided_rows_and_empty_group(gpu):
    rng = np.random.default_rng(9)
    big_a = torch.from_numpy(rng.integers(-2, 3, size=(96, 200)).astype(np.float32)).to(gpu).half()
    big_b = torch.from_numpy(rng.integers(-2, 3, size=(64, 400)).astype(np.float32)).to(gpu).half()
    a, b = big_a[:, :64], big_b[:, 8:136]          # lda = 200, ldb = 400 elements
    (c,) = triton_amd.group_gemm_fn([a], [b])
    assert torch.equal(c.float(), a.float() @ b.float())
    assert triton_amd.group_gemm_fn([], []) == []
    with pytest.raises(AssertionError):
        triton_amd.group_gemm_fn([a], [b, b])


@pytest.mark.parametrize("chunk", [4, 1, 3])
@pytest.mark.parametrize("nprog", [0, 7, 100])
def test_groups_of_whole_256_tiles(gpu, nprog, chunk, monkeypatch):
    # every problem whole 256x256 tiles and K % 128 == 0: the four-wave 16x16-MFMA kernel takes the group
    # (thresholds lowered so that 20 tiles and K = 128 are enough); exact sums of small integers, rounded
    # once; K from one pair of stages up to several, M != N, problems of one tile between larger ones
    set_knob(monkeypatch, "MI355_GROUPED_BIG_MIN", "1")
    set_knob(monkeypatch, "MI355_GROUPED_WAVE128_MIN_K", "128")
    # a program's tiles: chunks of up to 4 / 1 / 3 consecutive tiles (7 programs, 20 tiles: chunks of 3, runs that
    # cross from one problem into the next and runs of several tiles inside one problem)
    set_knob(monkeypatch, "MI355_GROUPED_CHUNK", str(chunk))
    rng = np.random.default_rng(40 + nprog)
    shapes = [(256, 256, 128), (512, 256, 256), (256, 256, 1024), (256, 768, 384), (1024, 512, 128), (256, 256, 256), (512, 512, 640)]
    ga = [rng.integers(-2, 3, size=(m, k)).astype(np.float32) for m, n, k in shapes]
    gb = [rng.integers(-2, 3, size=(k, n)).astype(np.float32) for m, n, k in shapes]
    ref = [a @ b for a, b in zip(ga, gb)]
    for dtype in ("fp16", "bf16"):
        outs = _run(gpu, ga, gb, dtype, num_programs=nprog)
        for c, r in zip(outs, ref):
            assert bits_equal(c, formats.round_to(r, dtype))   # (K = 1024 reaches beyond bf16's exact integers)
    # the same group through the eight-wave kernels
    set_knob(monkeypatch, "MI355_GROUPED_WAVE128_MIN_K", "0")
    for c, r in zip(_run(gpu, ga, gb, "fp16", num_programs=nprog), ref):
        assert bits_equal(c, r)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_whole_tile_groups_at_the_default_thresholds_against_closed_form(gpu, dtype):
    # 256 tiles of 256x256 with K = 2048 select the four-wave kernel without any knob: N(0,1) operands, padded
    # rows of A and C-sized B pitch of 512-byte multiples in the second problem.  A B pitch that is no such
    # multiple (third case) sends the group to the eight-wave kernels.
    rng = np.random.default_rng(5)
    mk = lambda shape: formats.round_to(rng.standard_normal(shape).astype(np.float32), dtype)
    a = [mk((2048, 2048)) for _ in range(4)]
    b = [mk((2048, 2048)) for _ in range(4)]
    ref = [gemm.matmul_closed_form(x, y, out_dtype=dtype) for x, y in zip(a, b)]
    ta = [from_np(x, dtype, gpu) for x in a]
    tb = [from_np(y, dtype, gpu) for y in b]
    ta[1] = from_np(np.pad(a[1], ((0, 0), (0, 64))), dtype, gpu)[:, :2048]
    for pad in (0, 256, 8):
        if pad:
            tb[1] = from_np(np.pad(b[1], ((0, 0), (pad, 0))), dtype, gpu)[:, pad:]
        outs = triton_amd.group_gemm_fn(ta, tb)
        for c, r in zip(outs, ref):
            assert np.allclose(to_np(c), r, rtol=1e-2, atol=1e-2), pad
            assert np.mean(to_np(c) == r) > 0.98
