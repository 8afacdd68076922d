"""CPU: block-scaled (MX) oracle.  The reference snapshot has no MX code: parity is pinned by
the OCP closed forms and exactness arguments only ("parity unpinned" by the reference)."""
import numpy as np

from oracle import formats, mx


def test_dequant_block_structure():
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 16, size=(4, 64)).astype(np.uint8)
    packed = formats.pack_fp4(codes)
    scales = np.array([[127, 128], [126, 127], [130, 120], [127, 127]], dtype=np.uint8)
    x = mx.mx_dequant(packed, scales, "mxfp4")
    tab = formats.e2m1_table().astype(np.float64)
    for r in range(4):
        for kb in range(2):
            exp = tab[codes[r, kb * 32:(kb + 1) * 32]] * 2.0 ** (int(scales[r, kb]) - 127)
            assert np.array_equal(x[r, kb * 32:(kb + 1) * 32], exp)


def test_matmul_exact_small_scales_any_order():
    # fp4 values are multiples of 0.5 up to 6; with scales in 2^-1..2^1 every product is a
    # multiple of 2^-4 below 144*... and partial sums over K <= 4096 stay exactly representable
    rng = np.random.default_rng(1)
    M, N, K = 24, 20, 256
    a = rng.integers(0, 256, size=(M, K // 2)).astype(np.uint8)
    b = rng.integers(0, 256, size=(N, K // 2)).astype(np.uint8)
    sa = rng.integers(126, 129, size=(M, K // 32)).astype(np.uint8)
    sb = rng.integers(126, 129, size=(N, K // 32)).astype(np.uint8)
    c = mx.mx_matmul(a, sa, b, sb, "mxfp4", out_dtype="fp32")
    # integer arithmetic in units of 2^-4: values*2 are integers, scales*2 are integers
    av = (formats.e2m1_table()[formats.unpack_fp4(a)] * 2).astype(np.int64) * np.repeat((2.0 ** (sa.astype(np.int64) - 126)).astype(np.int64), 32, axis=1)
    bv = (formats.e2m1_table()[formats.unpack_fp4(b)] * 2).astype(np.int64) * np.repeat((2.0 ** (sb.astype(np.int64) - 126)).astype(np.int64), 32, axis=1)
    exact = (av @ bv.T).astype(np.float64) / 16.0
    assert np.array_equal(c.astype(np.float64), exact)


def test_mxfp8_identity_scales_reduce_to_plain_fp8_matmul():
    rng = np.random.default_rng(2)
    M, N, K = 16, 12, 64
    a = rng.integers(0, 0x7F, size=(M, K)).astype(np.uint8)
    b = rng.integers(0, 0x7F, size=(N, K)).astype(np.uint8)
    one = np.full((M, K // 32), 127, np.uint8), np.full((N, K // 32), 127, np.uint8)
    c = mx.mx_matmul(a, one[0], b, one[1], "mxfp8", out_dtype="fp32")
    t = formats.fp8_table("e4m3").astype(np.float64)
    assert np.allclose(c, t[a] @ t[b].T, rtol=1e-6)
    # doubling one block scale of a row adds exactly that block's partial product once more
    sa2 = one[0].copy(); sa2[3, 1] = 128
    c2 = mx.mx_matmul(a, sa2, b, one[1], "mxfp8", out_dtype="fp32")
    extra = t[a[3, 32:64]] @ t[b[:, 32:64]].T
    assert np.allclose(c2[3] - c[3], extra, rtol=1e-5, atol=1e-3)
    assert np.array_equal(np.delete(c2, 3, axis=0), np.delete(c, 3, axis=0))
