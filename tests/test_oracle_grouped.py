"""Grouped-GEMM oracle (CPU): the tile walk of the reference kernel covers every tile exactly once
for any program count, and the tile-by-tile result equals the per-problem closed form."""
import numpy as np
import pytest

from oracle import gemm


@pytest.mark.parametrize("nprog", [1, 3, 84, 512])
def test_tile_walk_is_a_partition_of_all_tiles(nprog):
    sizes = [(1024, 1024, 1024), (512, 512, 512), (256, 256, 256), (128, 128, 128), (130, 70, 40), (1, 300, 8)]
    BM = BN = 128
    walks = gemm.grouped_tile_walk(sizes, BM, BN, nprog)
    seen = [t for w in walks for t in w]
    expect = [(g, tm, tn) for g, (m, n, _k) in enumerate(sizes)
              for tm in range(gemm.cdiv(m, BM)) for tn in range(gemm.cdiv(n, BN))]
    assert sorted(seen) == expect and len(seen) == len(set(seen))
    # program b starts at global tile b and strides by nprog: brute force over the flat numbering
    flat = {t: i for i, t in enumerate(expect)}
    for b, w in enumerate(walks):
        assert [flat[t] for t in w] == list(range(b, len(expect), nprog))


def test_grouped_result_equals_closed_form_and_is_exact_on_integers():
    rng = np.random.default_rng(3)
    shapes = [(256, 128, 64), (130, 70, 40), (1, 300, 8), (128, 128, 128)]
    ga = [rng.integers(-3, 4, size=(m, k)).astype(np.float32) for m, n, k in shapes]
    gb = [rng.integers(-3, 4, size=(k, n)).astype(np.float32) for m, n, k in shapes]
    outs = gemm.grouped_matmul(ga, gb, num_programs=7, out_dtype="fp32")
    for a, b, c in zip(ga, gb, outs):
        assert np.array_equal(c, (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32))
    # rounding point: one rounding of the fp32 accumulator to fp16
    fa = [rng.standard_normal((64, 96)).astype(np.float16).astype(np.float32)]
    fb = [rng.standard_normal((96, 32)).astype(np.float16).astype(np.float32)]
    out = gemm.grouped_matmul(fa, fb, out_dtype="fp16")[0]
    assert np.allclose(out, gemm.matmul_closed_form(fa[0], fb[0], out_dtype="fp16"), rtol=1e-2, atol=1e-2)
    assert np.array_equal(out, out.astype(np.float16).astype(np.float32))
