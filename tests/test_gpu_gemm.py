"""GPU parity: dense GEMM (fp16 / bf16 / fp8) through the C ABI against the CPU oracle.

Tolerances: rtol = atol = 1e-2 for fp16 / bf16 outputs, 3e-2 for fp8 inputs (the bar stated for
this build; the reference's own are atol 1e-2 at 512^3, python/tutorials/03-matrix-multiplication.py:368,
and rtol 1e-2 / atol 1e-3 vs an fp32 golden, python/test/unit/hopper/test_gemm.py:138-140);
bit-exact where every partial sum is exactly representable."""
import json
import os

import numpy as np
import pytest
import torch

import triton_amd
from triton_amd import _lib
from oracle import formats, gemm
from util import bits_equal, from_np, randn_rounded, report_error, to_np, set_knob

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
KAT = np.load(os.path.join(HERE, "golden", "gemm_kat.npz"))
GOLD_FMT = json.load(open(os.path.join(HERE, "golden", "formats.json")))


def test_config1_fp16_512_matches_tiled_oracle(gpu):
    # benchmark configuration 1: seed 0, 512^3 fp16, the oracle runs the reference tile program 64x64x32 / GROUP_M 8
    rng = np.random.default_rng(0)
    a = randn_rounded(rng, (512, 512), "fp16")
    b = randn_rounded(rng, (512, 512), "fp16")
    c = to_np(triton_amd.matmul(from_np(a, "fp16", gpu), from_np(b, "fp16", gpu)))
    ref = gemm.matmul_tiled(a, b, 64, 64, 32, 8, out_dtype="fp16")
    assert c.dtype == np.float32 and np.allclose(c, ref, rtol=1e-2, atol=1e-2)
    assert np.mean(c == ref) > 0.99  # same values except the odd fp16 tie
    assert np.allclose(c, gemm.matmul_closed_form(a, b, out_dtype="fp16"), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("layout", ["row_major_b", "k_major_b"])
@pytest.mark.parametrize("shape", [(256, 256, 64), (128, 128, 128), (300, 200, 136), (777, 1000, 520),
                                   (64, 8, 8), (1, 8, 8), (1024, 1024, 1024), (513, 264, 72)])
def test_shapes_and_layouts_against_closed_form(gpu, dtype, layout, shape):
    M, N, K = shape
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    a = randn_rounded(rng, (M, K), dtype)
    b = randn_rounded(rng, (K, N), dtype)
    ta = from_np(a, dtype, gpu)
    tb = from_np(b, dtype, gpu)
    if layout == "k_major_b":
        tb = tb.t().contiguous().t()   # same values, strides (1, K): the `b.T` view of 03:378-382
    c = to_np(triton_amd.matmul(ta, tb))
    ref = gemm.matmul_closed_form(a, b, out_dtype=dtype)
    assert np.allclose(c, ref, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("shape", [(100, 70, 50), (64, 64, 33), (37, 19, 7), (130, 250, 100)])
def test_unaligned_shapes_take_the_strided_kernel(gpu, shape):
    # K or N not a multiple of 8: no 16-byte rows, falls back to the strided kernel (still on the GPU)
    M, N, K = shape
    rng = np.random.default_rng(11)
    a = randn_rounded(rng, (M, K), "fp16")
    b = randn_rounded(rng, (K, N), "fp16")
    c = to_np(triton_amd.matmul(from_np(a, "fp16", gpu), from_np(b, "fp16", gpu)))
    assert np.allclose(c, gemm.matmul_tiled(a, b, 64, 64, 32, 8, out_dtype="fp16"), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", ["fp16", "bf16", "e4m3", "e5m2"])
def test_masked_mfma_kernel_against_the_fp32_fma_kernel_on_odd_shapes_and_strides(gpu, monkeypatch, dtype):
    # Operands that the tiled kernels do not take run 64 x 64 tiles on MFMAs with masked loads; the older kernel of fp32
    # FMAs (MI355_GEMM_FORCE_STRIDED=2) is a second implementation.  Integer-valued data: every sum is exact, so the
    # two - and the closed form - agree bit for bit, whatever the order of the sums.  Shapes with a single row or
    # column, K below and across the 32-element step, rows that start at odd addresses, B in all three layouts
    # (row-major, K-major, neither axis contiguous), C with a column stride.
    from triton_amd import _lib

    rng = np.random.default_rng(len(dtype) + ord(dtype[-1]))
    tdt = {"fp16": torch.float16, "bf16": torch.bfloat16, "e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}[dtype]
    abi = {"fp16": _lib.F16, "bf16": _lib.BF16, "e4m3": _lib.F8E4M3, "e5m2": _lib.F8E5M2}[dtype]
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    for (M, N, K) in [(1, 1, 1), (2047, 1, 1024), (1, 1100, 257), (100, 100, 512), (512, 33, 100), (65, 129, 31), (37, 19, 7),
                      (130, 250, 100), (64, 64, 33), (300, 70, 1000)]:
        a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
        ref = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)

        def dev(x):
            t = torch.from_numpy(x).to(gpu)
            return t.to(tdt)

        ta = dev(a)
        for layout in ("row-major", "K-major", "neither", "odd base"):
            if layout == "row-major":
                tb = dev(b)
            elif layout == "K-major":
                tb = dev(b).t().contiguous().t()
            elif layout == "neither":
                tb = torch.zeros(K, 3 * N, dtype=torch.float32, device=gpu).to(tdt)
                tb[:, ::3] = dev(b)
                tb = tb[:, ::3]
            else:
                flat = torch.zeros(K * N + 1, dtype=torch.float32, device=gpu).to(tdt)
                flat[1:] = dev(b).reshape(-1)
                tb = flat[1:].view(K, N)
            outs = []
            for force in ("1", "2"):
                set_knob(monkeypatch, "MI355_GEMM_FORCE_STRIDED", force)
                cbuf = torch.full((M, 2 * N), 7.0, dtype=torch.float32, device=gpu)
                c = cbuf[:, ::2]                                      # column stride 2
                rc = lib.mi355_gemm(ta.data_ptr(), tb.data_ptr(), c.data_ptr(), M, N, K, ta.stride(0), ta.stride(1),
                                    tb.stride(0), tb.stride(1), c.stride(0), c.stride(1), abi, _lib.F32, 0, 0, _lib.ACT_NONE, stream)
                assert rc == 0
                torch.cuda.synchronize()
                assert torch.all(cbuf[:, 1::2] == 7.0), "columns between the outputs untouched"
                outs.append(c.cpu().numpy())
            assert bits_equal(outs[0], ref), (dtype, M, N, K, layout)
            assert bits_equal(outs[1], ref), (dtype, M, N, K, layout, "fp32 FMA kernel")


def test_arbitrary_strides_on_b_and_c_views(gpu):
    rng = np.random.default_rng(12)
    a = randn_rounded(rng, (96, 64), "fp16")
    bbig = randn_rounded(rng, (64, 3 * 80), "fp16")
    tb = from_np(bbig, "fp16", gpu)[:, ::3]           # stride (240, 3): neither axis contiguous
    c = to_np(triton_amd.matmul(from_np(a, "fp16", gpu), tb))
    assert np.allclose(c, gemm.matmul_closed_form(a, bbig[:, ::3], out_dtype="fp16"), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("i", range(4))
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_golden_integer_cases_are_bit_exact(gpu, i, dtype):
    a, b, cgold = KAT[f"a{i}"].astype(np.float32), KAT[f"b{i}"].astype(np.float32), KAT[f"c{i}"].astype(np.float32)
    ta, tb = from_np(a, dtype, gpu), from_np(b, dtype, gpu)
    assert bits_equal(to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32)), cgold)
    assert bits_equal(to_np(triton_amd.matmul(ta, tb)), formats.round_to(cgold, dtype))
    tbk = tb.t().contiguous().t()
    assert bits_equal(to_np(triton_amd.matmul(ta, tbk, out_dtype=torch.float32)), cgold)


def test_exact_integers_on_mfma_path_bitwise_vs_tiled_oracle(gpu):
    # 16-byte aligned shapes so the MFMA kernels run; every partial sum is an exact integer
    rng = np.random.default_rng(5)
    for (M, N, K) in [(256, 256, 256), (384, 264, 200), (130, 72, 64)]:
        a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
        ref = gemm.matmul_tiled(a, b, 64, 64, 32, 8, out_dtype="fp32")
        for dtype in ("fp16", "bf16"):
            got = to_np(triton_amd.matmul(from_np(a, dtype, gpu), from_np(b, dtype, gpu), out_dtype=torch.float32))
            assert bits_equal(got, ref)


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5, 6])
def test_every_kernel_variant_is_bit_exact_on_integers(gpu, monkeypatch, tile):
    # MI355_GEMM_TILE forces one MFMA kernel (ping-pong, 128x128, one-barrier, pipelined 4 / 8 waves,
    # persistent, and 6 = four waves of 16x16x32 MFMAs for K-major B) for shapes the size heuristic would give to another; K = 520 has a
    # partial last K step, which the ping-pong kernel hands to the one-barrier kernel and the
    # pipelined kernels finish themselves; the persistent form takes whole tiles with K a multiple of
    # 128 (512 x 768 x 512 with 3 programs: two tiles each, in one stream of K steps) and falls back otherwise
    set_knob(monkeypatch, "MI355_GEMM_TILE", str(tile))
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", "3")
    rng = np.random.default_rng(11 + tile)
    for (M, N, K) in [(512, 768, 512), (300, 264, 520), (256, 256, 64), (1280, 1024, 128)]:
        a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
        ref = gemm.matmul_closed_form(a, b, out_dtype="fp32")
        for dtype in ("fp16", "bf16"):
            got = to_np(triton_amd.matmul(from_np(a, dtype, gpu), from_np(b, dtype, gpu), out_dtype=torch.float32))
            assert bits_equal(got, ref), (tile, dtype, M, N, K, "row-major B")
            bt = from_np(np.ascontiguousarray(b.T), dtype, gpu).t()  # K-major B
            got = to_np(triton_amd.matmul(from_np(a, dtype, gpu), bt, out_dtype=torch.float32))
            assert bits_equal(got, ref), (tile, dtype, M, N, K, "K-major B")
        # fp8: small integers are exact e4m3 / e5m2 values
        for fmt, tdt in (("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)):
            ca, cb = formats.encode_fp8(a, fmt), formats.encode_fp8(np.ascontiguousarray(b.T), fmt)
            got = to_np(triton_amd.matmul(torch.from_numpy(ca).to(gpu).view(tdt), torch.from_numpy(cb).to(gpu).view(tdt).t(),
                                          out_dtype=torch.float32))
            assert bits_equal(got, ref), (tile, fmt, M, N, K)


def test_single_nonzero_locates_every_tile(gpu):
    M, N, K = 520, 776, 136   # edge tiles for both tile sizes, K tail
    for (i, k, j) in [(0, 0, 0), (519, 135, 775), (255, 63, 256), (256, 64, 255), (300, 128, 511), (512, 7, 768)]:
        a = torch.zeros(M, K, dtype=torch.bfloat16, device=gpu); b = torch.zeros(K, N, dtype=torch.bfloat16, device=gpu)
        a[i, k] = 3.0; b[k, j] = -2.0
        c = triton_amd.matmul(a, b, out_dtype=torch.float32)
        nz = torch.nonzero(c)
        assert nz.tolist() == [[i, j]] and c[i, j].item() == -6.0


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_four_wave_16x16_kernel_against_closed_form(gpu, monkeypatch, dtype):
    # the 128x128-per-wave kernel of 16x16x32 MFMAs (K-major B, whole 256x256 tiles, K bytes % 256 == 0):
    # N(0,1) operands, every output type, alpha, the activation, a padded C, and the smallest K (two steps)
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    rng = np.random.default_rng(23)
    for (M, N, K) in [(512, 256, 1152), (256, 768, 128)]:
        a = randn_rounded(rng, (M, K), dtype)
        b = randn_rounded(rng, (K, N), dtype)
        ta = from_np(a, dtype, gpu)
        tb = from_np(np.ascontiguousarray(b.T), dtype, gpu).t()
        for out in ("fp32", dtype):
            odt = torch.float32 if out == "fp32" else ta.dtype
            c = to_np(triton_amd.matmul(ta, tb, out_dtype=odt))
            assert np.allclose(c, gemm.matmul_closed_form(a, b, out_dtype=out), rtol=1e-2, atol=1e-2), (M, N, K, out)
        c = to_np(triton_amd.matmul(ta, tb, activation="leaky_relu", a_scale=0.5, b_scale=4.0, out_dtype=torch.float32))
        ref = gemm.matmul_closed_form(a, b, out_dtype="fp32") * 2.0
        assert np.allclose(c, np.where(ref >= 0, ref, 0.01 * ref), rtol=1e-2, atol=1e-2)
        # the same product through the autotuner entry into a C with padded rows
        from triton_amd import autotune as at
        cbuf = torch.zeros(M, N + 8, device=gpu, dtype=ta.dtype)
        at._launch(ta, tb, cbuf[:, :N], at.Config(6, 4))
        assert np.allclose(to_np(cbuf[:, :N]), gemm.matmul_closed_form(a, b, out_dtype=dtype), rtol=1e-2, atol=1e-2)
        assert torch.count_nonzero(cbuf[:, N:]).item() == 0
        # and into a column-major C (unit stride along M: the epilogue falls back to single stores), row-major B
        ct = torch.zeros(N, M, device=gpu, dtype=torch.float32)
        at._launch(ta, from_np(b, dtype, gpu), ct.t(), at.Config(6, 8))
        assert np.allclose(to_np(ct.t()), gemm.matmul_closed_form(a, b, out_dtype="fp32"), rtol=1e-2, atol=1e-2)
        # row-major B as a column slice of wider matrices: a pitch that is a multiple of 512 bytes (this kernel)
        # and one that is not (its column-group XOR needs that multiple: another kernel takes the product)
        for pad in (256, 8):
            wide = from_np(np.pad(b, ((0, 0), (pad, pad))), dtype, gpu)
            c = to_np(triton_amd.matmul(ta, wide[:, pad:pad + N], out_dtype=torch.float32))
            assert np.allclose(c, gemm.matmul_closed_form(a, b, out_dtype="fp32"), rtol=1e-2, atol=1e-2), pad


@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_four_wave_16x16_fp8_kernel_against_dequantised_closed_form(gpu, monkeypatch, fmt, tdt):
    # the fp8 form of the same kernel (16x16x128 MFMAs; K-major B, whole tiles, K % 256 == 0): every finite
    # code as input, per-tensor scales, fp32 and bf16 outputs
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    rng = np.random.default_rng(29)
    table = formats.fp8_table(fmt)
    finite = np.array([c for c in range(256) if np.isfinite(table[c])], dtype=np.uint8)
    for (M, N, K) in [(256, 512, 768), (512, 256, 256)]:
        ca = rng.choice(finite, size=(M, K)); cb = rng.choice(finite, size=(N, K))
        a = table[ca].astype(np.float64); b = table[cb].astype(np.float64)
        # keep the products in range: scale both operands down by their largest magnitude
        sa, sb = 1.0 / np.abs(a).max(), 1.0 / np.abs(b).max()
        ref = (a @ b.T) * (sa * sb)
        ta = torch.from_numpy(ca).to(gpu).view(tdt); tb = torch.from_numpy(cb).to(gpu).view(tdt).t()
        got = to_np(triton_amd.matmul(ta, tb, a_scale=float(sa), b_scale=float(sb), out_dtype=torch.float32))
        assert np.allclose(got, ref, rtol=3e-2, atol=3e-2 * np.abs(ref).max()), (fmt, M, N, K)
        got = to_np(triton_amd.matmul(ta, tb, a_scale=float(sa), b_scale=float(sb), out_dtype=torch.bfloat16))
        assert np.allclose(got, ref, rtol=3e-2, atol=3e-2 * np.abs(ref).max()), (fmt, M, N, K, "bf16")


def test_leaky_relu_epilogue(gpu):
    rng = np.random.default_rng(6)
    a = randn_rounded(rng, (256, 128), "fp16"); b = randn_rounded(rng, (128, 264), "fp16")
    c = to_np(triton_amd.matmul(from_np(a, "fp16", gpu), from_np(b, "fp16", gpu), activation="leaky_relu"))
    assert np.allclose(c, gemm.matmul_tiled(a, b, 64, 64, 32, 8, activation="leaky_relu", out_dtype="fp16"), rtol=1e-2, atol=1e-2)
    with pytest.raises(KeyError):
        triton_amd.matmul(from_np(a, "fp16", gpu), from_np(b, "fp16", gpu), activation="gelu")


@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
@pytest.mark.parametrize("shape", [(128, 128, 128), (512, 512, 512), (300, 200, 144), (16, 1024, 2048), (1024, 1024, 1024)])
def test_fp8_against_dequantised_closed_form(gpu, fmt, tdt, shape):
    # config 4 construction: x / (amax/448) cast to fp8, per-tensor fp32 scales, bf16 out = acc * sa * sb
    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    xa = rng.standard_normal((M, K)).astype(np.float32)
    xb = rng.standard_normal((N, K)).astype(np.float32)
    fmax = formats.fp8_table(fmt)[formats.FP8_FORMATS[fmt][3]]
    sa, sb = np.abs(xa).max() / fmax, np.abs(xb).max() / fmax
    ca, cb = formats.encode_fp8(xa / sa, fmt), formats.encode_fp8(xb / sb, fmt)
    ta = torch.from_numpy(ca).to(gpu).view(tdt)
    tb = torch.from_numpy(cb).to(gpu).view(tdt)            # stored [N, K], passed as the .T view
    tab = formats.fp8_table(fmt)
    ref = gemm.matmul_closed_form(tab[ca], tab[cb].T, out_dtype="bf16", alpha=float(sa) * float(sb))
    c = to_np(triton_amd.matmul(ta, tb.t(), out_dtype=torch.bfloat16,
                                a_scale=torch.tensor([sa], device=gpu), b_scale=float(sb)))
    assert np.allclose(c, ref, rtol=3e-2, atol=3e-2)
    # default output type for fp8 inputs is fp16, as in the reference (03:337); unscaled N(0,1) codes
    # keep the products inside the fp16 range
    da, db = formats.encode_fp8(xa, fmt), formats.encode_fp8(xb, fmt)
    c16 = triton_amd.matmul(torch.from_numpy(da).to(gpu).view(tdt), torch.from_numpy(db).to(gpu).view(tdt).t())
    assert c16.dtype == torch.float16
    assert np.allclose(to_np(c16), gemm.matmul_closed_form(tab[da], tab[db].T, out_dtype="fp16"), rtol=3e-2, atol=3e-2)


def test_fp8_raw_code_inputs_like_reference_test(gpu):
    # test_core.py:5109-5176: 128x256x256, raw codes randint(20, 40), reference = matmul of the upcast values
    rng = np.random.RandomState(17)
    ca = rng.randint(20, 40, size=(128, 256)).astype(np.uint8)
    cb = rng.randint(20, 40, size=(256, 256)).astype(np.uint8)   # [N, K]
    tab = formats.fp8_table("e4m3")
    ref = gemm.matmul_closed_form(tab[ca], tab[cb].T, out_dtype="fp32")
    c = to_np(triton_amd.matmul(torch.from_numpy(ca).to(gpu).view(torch.float8_e4m3fn),
                                torch.from_numpy(cb).to(gpu).view(torch.float8_e4m3fn).t(), out_dtype=torch.float32))
    assert np.allclose(c, ref, rtol=0.01, atol=0.01)


def test_fp8_row_major_b_of_unaligned_rows_and_fp8_output(gpu):
    # (rows of 72 bytes are not whole 16-byte chunks: the strided kernel, whose sums are in fp32 order of k)
    rng = np.random.default_rng(8)
    ca = formats.encode_fp8(rng.standard_normal((64, 96)).astype(np.float32), "e4m3")
    cb = formats.encode_fp8(rng.standard_normal((96, 72)).astype(np.float32), "e4m3")    # [K, N] row-major
    tab = formats.fp8_table("e4m3")
    ta = torch.from_numpy(ca).to(gpu).view(torch.float8_e4m3fn)
    tb = torch.from_numpy(cb).to(gpu).view(torch.float8_e4m3fn)
    ref = gemm.matmul_closed_form(tab[ca], tab[cb], out_dtype="fp32")
    assert np.allclose(to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32)), ref, rtol=1e-3, atol=1e-3)
    # tutorial 09 `matmul`: result dtype = input dtype (09:93-96, :124)
    out8 = triton_amd.matmul_like_input(ta, tb)
    assert out8.dtype == torch.float8_e4m3fn
    assert np.array_equal(out8.view(torch.uint8).cpu().numpy(), formats.encode_fp8(ref, "e4m3"))
    a16 = from_np(tab[ca], "fp16", gpu); b16 = from_np(tab[cb], "fp16", gpu)
    assert triton_amd.matmul_like_input(a16, b16).dtype == torch.float16


@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
@pytest.mark.parametrize("shape", [(128, 128, 64), (256, 256, 256), (300, 208, 144), (100, 16, 48), (512, 768, 1040), (1024, 2048, 512),
                                   (2304, 2560, 320)])
def test_row_major_fp8_b_runs_the_mfma_kernels_bit_exactly(gpu, fmt, tdt, shape):
    # `matmul(a, b)` with b stored [K, N] (what tutorial 03 passes before its fp8 special case, 03:378-380): the C ABI
    # transposes the B tile on its way out of LDS.  Small integers as operands: every sum is exact in fp32, so the
    # product equals numpy's and the K-major call's bit for bit - edge tiles, K tails (K % 64 != 0) and both tile sizes.
    M, N, K = shape
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    xa = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    xb = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
    ta = torch.from_numpy(formats.encode_fp8(xa, fmt)).to(gpu).view(tdt)
    tb = torch.from_numpy(formats.encode_fp8(xb, fmt)).to(gpu).view(tdt)                   # [K, N] row-major
    got = triton_amd.matmul(ta, tb, out_dtype=torch.float32)
    assert np.array_equal(to_np(got), xa.astype(np.float64) @ xb.astype(np.float64))
    assert torch.equal(got, triton_amd.matmul(ta, tb.t().contiguous().t(), out_dtype=torch.float32))
    # a pitch wider than the row (a column slice of a larger matrix)
    wide = torch.zeros(K, N + 48, dtype=torch.uint8, device=gpu).view(tdt)
    wide[:, 16:16 + N] = tb
    assert torch.equal(triton_amd.matmul(ta, wide[:, 16:16 + N], out_dtype=torch.float32), got)


@pytest.mark.parametrize("programs", [3, 256])
@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_four_wave_fp8_kernel_with_a_row_major_b_is_bit_exact(gpu, monkeypatch, fmt, tdt, programs):
    # the four-wave fp8 kernel's form for B[K, N]: 128 k rows of 256 bytes per stage, fragments by 8-bit transpose reads.
    # Whole tiles and pairs of K steps; one and several tiles per program; every epilogue the form has (fp32: general;
    # fp16, bf16: lean); a pitch wider than the row.  Integer data: the bits of the exact product and of the K-major call.
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", programs)
    rng = np.random.default_rng(programs + len(fmt))
    for (M, N, K, pad) in [(256, 256, 256, 0), (768, 512, 512, 0), (512, 768, 1280, 64), (256, 1024, 2048, 16)]:
        a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
        b = rng.integers(-3, 4, size=(K, N)).astype(np.float32)
        ta = torch.from_numpy(formats.encode_fp8(a, fmt)).to(gpu).view(tdt)
        wide = torch.zeros(K, N + pad, dtype=torch.uint8, device=gpu).view(tdt)
        wide[:, :N] = torch.from_numpy(formats.encode_fp8(b, fmt)).to(gpu).view(tdt)
        tb = wide[:, :N]                                                                    # [K, N], pitch N + pad
        want = a.astype(np.float64) @ b.astype(np.float64)
        got32 = triton_amd.matmul(ta, tb, out_dtype=torch.float32)
        assert np.array_equal(to_np(got32), want), (M, N, K, fmt, programs)
        assert torch.equal(got32, triton_amd.matmul(ta, tb.t().contiguous().t(), out_dtype=torch.float32))
        for out, name in ((torch.float16, "fp16"), (torch.bfloat16, "bf16")):
            got = to_np(triton_amd.matmul(ta, tb, out_dtype=out))
            assert bits_equal(got, gemm.matmul_closed_form(a, b, out_dtype=name)), (M, N, K, fmt, programs, name)


def test_large_row_major_fp8_b_runs_on_the_fp8_mfmas_inside_the_c_abi(gpu):
    # 03:378-380 pre-transposes b on the host for fp8; here mi355_gemm itself takes the row-major B (no copy of B in
    # the wrapper): told apart from the strided kernel by time, equal to the K-major call bit for bit (the same
    # products summed in the same order: both forms walk K in 64-byte steps with the same lane assignment)
    n = 4096
    g = torch.Generator(device="cpu").manual_seed(12)
    a = (torch.randn(n, n, generator=g) * 0.5).to(torch.float8_e4m3fn).to(gpu)
    b = (torch.randn(n, n, generator=g) * 0.5).to(torch.float8_e4m3fn).to(gpu)     # [K, N] row-major
    got = torch.empty(n, n, dtype=torch.bfloat16, device=gpu)
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream

    def call():
        rc = lib.mi355_gemm(a.data_ptr(), b.data_ptr(), got.data_ptr(), n, n, n, a.stride(0), a.stride(1), b.stride(0), b.stride(1),
                            got.stride(0), got.stride(1), _lib.F8E4M3, _lib.BF16, None, None, _lib.ACT_NONE, stream)
        assert rc == 0, rc

    call()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    call()
    ev1.record()
    torch.cuda.synchronize()
    ms = ev0.elapsed_time(ev1)
    print(f"mi355_gemm, row-major e4m3 B, 4096^3: {ms:.3f} ms = {2 * n ** 3 / ms / 1e9:.0f} TFLOP/s")
    assert ms < 1.0, ms
    rows = [0, 255, 2048, 4095]
    ref = a[rows].double() @ b.double()
    err = (got[rows].double() - ref).abs().max().item()
    print(f"max abs error against fp64 on 4 rows: {err:.3e}")
    assert torch.allclose(got[rows].double(), ref, rtol=1e-2, atol=0.02)      # (bf16 results: half an ulp is 2^-9 of the value)
    assert torch.equal(triton_amd.matmul(a, b, out_dtype=torch.bfloat16), got)


@pytest.mark.parametrize("tile", [None, 6])
@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_fp8_output_of_the_mfma_epilogues_rounds_like_the_oracle(gpu, monkeypatch, fmt, tdt, tile):
    # fp8 outputs (tutorial 09: c has the dtype of a, 09:93-96, :124) are stored by the MFMA kernels' own
    # epilogues.  A zero product plus an fp32 addend puts chosen fp32 values through that conversion: every
    # code value, every midpoint between neighbouring codes (ties to even), values just off the midpoints,
    # sub-normal results, finite overflow (saturates to the largest finite code) and NaN.
    if tile is not None:
        set_knob(monkeypatch, "MI355_GEMM_TILE", tile)     # 6: four-wave kernel (its own epilogue); default here: 128x128 tiles
    n = 512
    tab = formats.fp8_table(fmt).astype(np.float64)
    _, _, _, max_code = formats.FP8_FORMATS[fmt]
    pos = tab[: max_code + 1]
    mids = (pos[:-1] + pos[1:]) / 2
    vals = np.concatenate([pos, mids, mids * (1 + 2.0 ** -20), mids * (1 - 2.0 ** -20), [pos[-1] * 1.01, pos[-1] * 1.07, 1e9, 3e38],
                           [pos[1] / 2, pos[1] / 4, pos[1] * 0.75, 1e-30]])
    vals = np.concatenate([vals, -vals]).astype(np.float32)
    rng = np.random.default_rng(3)
    d = np.concatenate([vals, (rng.standard_normal(n * n - len(vals) - 2) * 30).astype(np.float32), [np.nan, -np.nan]]).astype(np.float32)
    d = d.reshape(n, n)
    z = torch.zeros(n, n, dtype=torch.bfloat16, device=gpu)
    out = triton_amd.matmul(z, z, add=torch.from_numpy(d).to(gpu), out_dtype=tdt)
    got = out.view(torch.uint8).cpu().numpy()
    want = formats.encode_fp8(d, fmt)
    finite = ~np.isnan(d)
    assert np.array_equal(got[finite] & 0x7F, want[finite] & 0x7F)
    nz = finite & (want & 0x7F != 0)
    assert np.array_equal(got[nz] >> 7, want[nz] >> 7)                      # sign (of non-zero results)
    assert np.all(np.isnan(formats.fp8_table(fmt)[got[~finite]]))           # NaN stays NaN


def test_full_size_fp8_to_fp8_runs_an_mfma_kernel(gpu):
    # tutorial 09's matmul on e4m3fn operands returns e4m3fn (09:105-138): at 8192^3 that must be the
    # four-wave MFMA kernel, not the one-thread-per-output strided kernel - told apart by time (the strided
    # kernel needs seconds for this product)
    n = 8192
    g = torch.Generator(device="cpu").manual_seed(9)
    a = (torch.randn(n, n, generator=g) * 0.25).to(torch.float8_e4m3fn)
    b = (torch.randn(n, n, generator=g) * 0.25).to(torch.float8_e4m3fn)     # [N, K]
    ta, tb = a.to(gpu), b.to(gpu).t()
    out = triton_amd.matmul_like_input(ta, tb)
    assert out.dtype == torch.float8_e4m3fn
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(3):
        out = triton_amd.matmul_like_input(ta, tb)
    ev1.record()
    torch.cuda.synchronize()
    ms = ev0.elapsed_time(ev1) / 3
    print(f"fp8 -> fp8 8192^3: {ms:.3f} ms per call")
    assert ms < 5.0, ms
    rows = [0, 255, 4096, 8191]
    ref = a[rows].double().numpy() @ b.double().numpy().T
    tab = formats.fp8_table("e4m3")
    got = tab[out[rows].view(torch.uint8).cpu().numpy()]
    want = tab[formats.encode_fp8(ref.astype(np.float32), "e4m3")]
    # the fp8 MFMA's accumulation error (about 6e-5 relative) may move a value across a rounding boundary:
    # equal codes almost everywhere, never more than one code apart (e4m3 spacing: 2^-3 relative)
    assert np.mean(got == want) > 0.98
    assert np.allclose(got, want, rtol=0.13, atol=2.0 ** -9)
    assert np.allclose(got, ref, rtol=0.07, atol=2.0 ** -9)                  # half a code spacing (plus slack) from the exact product


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1", "e8m0"])
def test_dequant_tables_bit_exact(gpu, fmt):
    n = 16 if fmt == "e2m1" else 256
    gold = np.array(GOLD_FMT[fmt], dtype=np.uint32)
    if fmt == "e2m1":
        codes = torch.tensor([lo | (hi << 4) for lo, hi in zip(range(0, 16, 2), range(1, 16, 2))], dtype=torch.uint8, device=gpu)
    else:
        codes = torch.arange(256, dtype=torch.uint8, device=gpu)
    out = triton_amd.dequantize(codes, fmt).cpu().numpy().view(np.uint32)
    nan = (gold & 0x7FFFFFFF) > 0x7F800000
    assert out.shape == (n,) and np.array_equal(out[~nan], gold[~nan])
    assert np.all((out[nan] & 0x7FFFFFFF) > 0x7F800000)


@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_mfma_decodes_every_fp8_code_exactly(gpu, fmt, tdt):
    # A[m, 0] = code m, B = e_0 * 1.0: C[m, 0] is the hardware's decode of code m
    tab = formats.fp8_table(fmt)
    codes = np.array([c for c in range(256) if np.isfinite(tab[c])], dtype=np.uint8)
    a = np.zeros((256, 128), np.uint8); a[: len(codes), 0] = codes
    b = np.zeros((128, 128), np.uint8); b[0, 0] = formats.encode_fp8(np.array([1.0], np.float32), fmt)[0]
    c = to_np(triton_amd.matmul(torch.from_numpy(a).to(gpu).view(tdt), torch.from_numpy(b).to(gpu).view(tdt).t(),
                                out_dtype=torch.float32))
    assert bits_equal(np.abs(c[: len(codes), 0]), np.abs(tab[codes]))   # sign of zero aside
    assert np.array_equal(np.sign(c[: len(codes), 0]), np.sign(tab[codes]))


def test_full_size_8192_bf16_sampled_rows_and_exact_permutation(gpu):
    # benchmark configuration 2 at full size: (a) sampled rows against the fp64 closed form, (b) B = signed
    # permutation makes every output one exactly-representable product -> bitwise
    n = 8192
    g = torch.Generator(device="cpu").manual_seed(0)
    a = torch.randn(n, n, generator=g).bfloat16()
    b = torch.randn(n, n, generator=g).bfloat16()
    c = triton_amd.matmul(a.to(gpu), b.to(gpu))
    assert c.dtype == torch.bfloat16
    rows = [0, 1, 255, 256, 4095, 4096, 8191, 5000]
    ref = formats.round_bf16((a[rows].double().numpy() @ b.double().numpy()).astype(np.float32))
    assert np.allclose(to_np(c[rows]), ref, rtol=1e-2, atol=1e-2)
    perm = torch.randperm(n, generator=g)
    sign = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).bfloat16()
    pb = torch.zeros(n, n, dtype=torch.bfloat16)
    pb[perm, torch.arange(n)] = sign                     # column j picks row perm[j] of B-as-K
    cp = triton_amd.matmul(a.to(gpu), pb.to(gpu)).cpu()
    assert torch.equal(cp, a[:, perm] * sign[None, :])
    # linearity in B at full size: A (b1 + b2) = A b1 + A b2 for exactly-summable b2 = -b1 + pb
    del c, cp


def _sampled_rows_check(gpu, M, N, K, dtype, seed, layout="row_major_b"):
    """C = A @ B at full size on N(0, 1) operands; rows at tile edges and a few inside are compared with the
    fp64 product rounded to the output type at rtol = atol = 1e-2, and one signed-permutation product
    (every output a single exactly representable term) bitwise."""
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    g = torch.Generator(device="cpu").manual_seed(seed)
    a = torch.randn(M, K, generator=g).to(tdt)
    b = torch.randn(K, N, generator=g).to(tdt)
    tb = b.to(gpu)
    if layout == "k_major_b":
        tb = tb.t().contiguous().t()
    c = triton_amd.matmul(a.to(gpu), tb)
    assert c.dtype == tdt and c.shape == (M, N)
    rows = sorted({0, 1, 255, 256, M // 2 - 1, M // 2, M - 257, M - 256, M - 1, (5 * M) // 8 + 3})
    ref = formats.round_to((a[rows].double().numpy() @ b.double().numpy()).astype(np.float32), dtype)
    got = to_np(c[rows])
    print(f"{M}x{N}x{K} {dtype} {layout}: max |err| {np.abs(got - ref).max():.3e} on {len(rows)} rows")
    assert np.allclose(got, ref, rtol=1e-2, atol=1e-2)
    if K <= N:
        perm = torch.randperm(N, generator=g)[:K] if K < N else torch.randperm(N, generator=g)
        sign = (torch.randint(0, 2, (K,), generator=g) * 2 - 1).to(tdt)
        pb = torch.zeros(K, N, dtype=tdt)
        pb[torch.arange(K), perm] = sign                 # row k of B has its one entry in column perm[k]
        cp = triton_amd.matmul(a.to(gpu), pb.to(gpu)).cpu()
        want = torch.zeros(M, N, dtype=tdt)
        want[:, perm] = a * sign[None, :]
        assert torch.equal(cp, want)


@pytest.mark.parametrize("n", [2048, 3072, 4096, 5120, 6144, 7168])
def test_config2_sweep_sizes_bf16(gpu, n):
    # benchmark configuration 2 sweeps square sizes 1024 .. 8192 (1024 and 8192 have tests of their own): 5120, 6144
    # and 7168 are the sizes whose tiles do not divide by the CU count, so the persistent programs walk ragged
    # rounds of tiles as one stream of K steps
    _sampled_rows_check(gpu, n, n, n, "bf16", seed=n)


def test_full_size_8192_fp16_sampled_rows(gpu):
    # config 2 names fp16 next to bf16
    _sampled_rows_check(gpu, 8192, 8192, 8192, "fp16", seed=5)


@pytest.mark.parametrize("programs", [3, 256])
@pytest.mark.parametrize("layout", ["row_major_b", "k_major_b"])
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_four_wave_kernel_k_tails_are_bit_exact(gpu, monkeypatch, dtype, layout, programs):
    # K not a multiple of 128 elements in the four-wave kernel: the rest (8 .. 120 elements) is multiplied after the
    # pipelined K loop through a buffer of its own, 32 elements at a time.  Every tail length class (one to four
    # half-steps, full and partial last one), one and several tiles per program (the tail runs while the stages
    # already hold the next tile's first K steps), integer data: the bits of the closed form.
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", programs)
    rng = np.random.default_rng(programs + len(layout))
    for K in (136, 264, 312, 376, 440, 504, 1016, 2056):
        M, N = 768, 512
        a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
        ta, tb = from_np(a, dtype, gpu), from_np(b, dtype, gpu)
        if layout == "k_major_b":
            tb = tb.t().contiguous().t()
        got = to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32))
        assert bits_equal(got, gemm.matmul_closed_form(a, b, out_dtype="fp32")), (K, dtype, layout, programs)
        # C in the operands' own type: the form of the four-wave kernel that has the tail (the fp32 output above is
        # another kernel's); the exact integer sums, rounded once
        own = to_np(triton_amd.matmul(ta, tb))
        assert bits_equal(own, gemm.matmul_closed_form(a, b, out_dtype=dtype)), (K, dtype, layout, programs, "own type")


@pytest.mark.parametrize("programs", [3, 256])
@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_four_wave_fp8_kernel_k_tails_are_bit_exact(gpu, monkeypatch, fmt, tdt, programs):
    # K bytes not a multiple of 256 in the four-wave fp8 kernel: what is left behind the last pair of 128-byte K steps
    # (16 .. 240 bytes) follows as one or two steps whose fragments come straight from global memory, zeros beyond K.
    # Every class of tail (one and two steps; a lane group's first chunk only, both, neither), one and several tiles
    # per program (the tail runs while the stages and half of the fragment registers already hold the next tile's
    # first K steps), every epilogue that has the form (fp32: general; fp16, bf16: lean).  Integer data: exact sums.
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", programs)
    rng = np.random.default_rng(programs + len(fmt))
    M, N = 768, 512
    for K in (272, 320, 336, 384, 400, 448, 496, 1008, 2064):
        a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
        b = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
        ta = torch.from_numpy(formats.encode_fp8(a, fmt)).to(gpu).view(tdt)
        tb = torch.from_numpy(formats.encode_fp8(b, fmt)).to(gpu).view(tdt).t()          # K-major B
        want = a.astype(np.float64) @ b.astype(np.float64).T
        assert np.array_equal(to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32)), want), (K, fmt, programs)
        for out, name in ((torch.float16, "fp16"), (torch.bfloat16, "bf16")):
            got = to_np(triton_amd.matmul(ta, tb, out_dtype=out))
            assert bits_equal(got, gemm.matmul_closed_form(a, b.T, out_dtype=name)), (K, fmt, programs, name)


@pytest.mark.parametrize("layout", ["row_major_b", "k_major_b"])
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_uneven_k_8192x8192x8176(gpu, dtype, layout):
    # the reference's own EVEN_K == False performance shape (python/test/regression/test_performance.py:46)
    _sampled_rows_check(gpu, 8192, 8192, 8176, dtype, seed=46, layout=layout)


def test_full_size_8192_fp8_sampled_rows_and_k_major_bf16(gpu):
    # benchmark configuration 4 at full size (e4m3fn codes with per-tensor scales, bf16 out), sampled rows against the
    # dequantised fp64 product; and config 2 with B stored K-major (the `b.T` view), sampled rows
    n = 8192
    g = torch.Generator(device="cpu").manual_seed(1)
    x = torch.randn(n, n, generator=g); y = torch.randn(n, n, generator=g)
    sx = (x.abs().amax() / 448).item(); sy = (y.abs().amax() / 448).item()
    qa = (x / sx).clamp(-448, 448).to(torch.float8_e4m3fn); qb = (y / sy).clamp(-448, 448).to(torch.float8_e4m3fn)   # qb is [N, K]
    c = triton_amd.matmul(qa.to(gpu), qb.to(gpu).t(), a_scale=sx, b_scale=sy, out_dtype=torch.bfloat16)
    rows = [0, 255, 256, 4097, 8191]
    ref = (qa[rows].double().numpy() @ qb.double().numpy().T) * (sx * sy)
    # (the working bar for fp8 is rtol = 3e-2; the absolute term, a 500th of the largest output, only covers outputs near 0)
    report_error("fp8 e4m3 8192^3, bf16 out, 5 rows", to_np(c[rows]), ref)
    assert np.allclose(to_np(c[rows]), ref, rtol=3e-2, atol=3e-2 * np.abs(ref).max() / 16)
    a16 = x.bfloat16(); b16 = y.bfloat16()                       # b16 is [N, K]: K-major B
    c16 = triton_amd.matmul(a16.to(gpu), b16.to(gpu).t())
    ref16 = formats.round_bf16((a16[rows].double().numpy() @ b16.double().numpy().T).astype(np.float32))
    assert np.allclose(to_np(c16[rows]), ref16, rtol=1e-2, atol=1e-2)


def test_decode_shape_m16(gpu):
    # config 4 decode variant: M = 16, N = K = 8192 (bandwidth bound)
    rng = np.random.default_rng(3)
    ca = formats.encode_fp8(rng.standard_normal((16, 8192)).astype(np.float32), "e4m3")
    cb = formats.encode_fp8(rng.standard_normal((8192, 8192)).astype(np.float32), "e4m3")
    tab = formats.fp8_table("e4m3")
    ref = gemm.matmul_closed_form(tab[ca], tab[cb].T, out_dtype="bf16")
    c = to_np(triton_amd.matmul(torch.from_numpy(ca).to(gpu).view(torch.float8_e4m3fn),
                                torch.from_numpy(cb).to(gpu).view(torch.float8_e4m3fn).t(), out_dtype=torch.bfloat16))
    assert np.allclose(c, ref, rtol=3e-2, atol=3e-2)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("shape", [(16, 256, 512), (64, 128, 1024), (33, 96, 64), (1, 32, 32), (7, 2048, 4096),
                                   (256, 64, 512), (128, 32, 256), (1024, 16, 2048), (96, 40, 96),
                                   (100, 2048, 512), (128, 2048, 256), (65, 4096, 128), (2048, 128, 512), (2048, 96, 256),
                                   (2048, 100, 256)])
def test_skinny_16bit_kernel_is_bit_exact_on_integers(gpu, monkeypatch, dtype, shape):
    # at most 64 rows on one side (shapes of python/test/regression/test_performance.py:36-44): the
    # streaming kernel (K split over the waves of a workgroup) for row-major and K-major B; M > 64
    # with N <= 64 takes it with the operands swapped (a row-major B then needs N = 32 or 64; the
    # other cases here fall through to the tile kernels); 65 .. 128 rows against at least 2048 on the other
    # side run as two launches, 64 rows and the rest.  Every partial sum is an exact integer,
    # so the result does not depend on how K is split.
    M, N, K = shape
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
    ref = gemm.matmul_closed_form(a, b, out_dtype="fp32")
    ta = from_np(a, dtype, gpu)
    for tb in (from_np(b, dtype, gpu), from_np(np.ascontiguousarray(b.T), dtype, gpu).t()):
        got = to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32))
        assert bits_equal(got, ref), (dtype, shape, tb.stride())
        set_knob(monkeypatch, "MI355_GEMM_SKINNY", "0")      # the tile kernels on the same inputs
        assert bits_equal(to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32)), ref)
        monkeypatch.delenv("MI355_GEMM_SKINNY")
    if dtype == "fp16":
        # fp8 (K-major B, the `b.T` view): the same streaming kernel with one 32x32x64 MFMA per stage
        for fmt, tdt in (("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)):
            ca, cb = formats.encode_fp8(a, fmt), formats.encode_fp8(np.ascontiguousarray(b.T), fmt)
            t8a, t8b = torch.from_numpy(ca).to(gpu).view(tdt), torch.from_numpy(cb).to(gpu).view(tdt).t()
            assert bits_equal(to_np(triton_amd.matmul(t8a, t8b, out_dtype=torch.float32)), ref), (fmt, shape)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_skinny_16bit_decode_shapes_against_closed_form(gpu, dtype):
    # M = 16 and 64 against N = K = 4096, and the transposed 4096 x 64: random data, output in the
    # input type, leaky-ReLU epilogue on one of them
    rng = np.random.default_rng(21)
    for (M, N, K), act in (((16, 4096, 4096), ""), ((64, 4096, 4096), "leaky_relu"), ((4096, 64, 4096), "")):
        a = randn_rounded(rng, (M, K), dtype)
        b = randn_rounded(rng, (K, N), dtype)
        ref = gemm.matmul_closed_form(a, b, out_dtype=dtype, activation=act)
        tb = from_np(b, dtype, gpu)
        c = to_np(triton_amd.matmul(from_np(a, dtype, gpu), tb, activation=act))
        assert np.allclose(c, ref, rtol=1e-2, atol=1e-2), (M, N, K, "row-major B")
        c = to_np(triton_amd.matmul(from_np(a, dtype, gpu), tb.t().contiguous().t(), activation=act))
        assert np.allclose(c, ref, rtol=1e-2, atol=1e-2), (M, N, K, "K-major B")


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_fused_addends_in_the_four_wave_kernel(gpu, dtype, monkeypatch):
    # the add-matrix / add-rows / add-cols forms (python/test/unit/language/test_core.py:3128-3145) in the
    # addend instantiation of the 16x16-MFMA kernel: integer data, bit-exact; both B layouts, addend in fp32
    # and in the input type, with scales and the activation, result in fp32 and in the input type
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    M, N, K = 512, 768, 256
    rng = np.random.default_rng(77)
    a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
    z = rng.integers(-4, 5, size=(M, N)).astype(np.float32)
    ta = from_np(a, dtype, gpu)
    for tb in (from_np(b, dtype, gpu), from_np(np.ascontiguousarray(b.T), dtype, gpu).t()):
        for add_dt in ("fp32", dtype):
            tz = from_np(z, add_dt, gpu)
            for add_np, add_t in ((z, tz), (z[:, :1], tz[:, :1]), (z[:1, :], tz[:1, :]), (z[0], tz[0])):
                got = to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32, add=add_t))
                assert bits_equal(got, gemm.dot_epilogue(a, b, add=add_np)), (dtype, add_dt, add_np.shape)
        got = to_np(triton_amd.matmul(ta, tb, add=from_np(z, "fp32", gpu), activation="leaky_relu", a_scale=0.5, b_scale=0.25))
        ref = a @ b * 0.125 + z
        ref = formats.round_to(np.where(ref >= 0, ref, np.float32(0.01) * ref).astype(np.float32), dtype)
        assert np.allclose(got, ref, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("programs", [2, 3, 4])
def test_four_wave_kernels_deal_tiles_in_ragged_rounds(gpu, monkeypatch, programs):
    # five tiles (1280 x 256) on at most 2 / 3 / 4 programs: 3 rounds on 2 programs (2 + 2 + 1 tiles), 2 rounds
    # on 3 (2 + 2 + 1) - with 4 CUs also 2 rounds, so again 3 programs; a program with fewer tiles than the others
    # wraps its loads earlier.  bf16 with both B layouts and fp8, sums of small integers: bit-exact.
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", str(programs))
    rng = np.random.default_rng(90 + programs)
    M, N = 1280, 256
    for K in (128, 384):
        a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
        ref = a @ b
        ta = from_np(a, "bf16", gpu)
        for tb in (from_np(b, "bf16", gpu), from_np(np.ascontiguousarray(b.T), "bf16", gpu).t()):
            assert bits_equal(to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32)), ref), (K, programs)
    K = 512
    a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
    ca, cb = formats.encode_fp8(a, "e4m3"), formats.encode_fp8(np.ascontiguousarray(b.T), "e4m3")
    t8a = torch.from_numpy(ca).to(gpu).view(torch.float8_e4m3fn)
    t8b = torch.from_numpy(cb).to(gpu).view(torch.float8_e4m3fn).t()
    assert bits_equal(to_np(triton_amd.matmul(t8a, t8b, out_dtype=torch.float32)), a @ b), programs


@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_fused_addends_in_the_four_wave_fp8_kernel(gpu, monkeypatch, fmt, tdt):
    # the same addend forms in the fp8 kernel of 16x16x128 MFMAs: codes of small integers (exact products
    # and sums), addend in fp32 and bf16, bit-exact in fp32
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    M, N, K = 512, 256, 512
    rng = np.random.default_rng(78)
    table = formats.fp8_table(fmt)
    small = np.array([c for c in range(256) if table[c] in (-2.0, -1.0, 0.0, 1.0, 2.0) and not (c == 0x80)], dtype=np.uint8)
    ca = rng.choice(small, size=(M, K)); cb = rng.choice(small, size=(N, K))
    a = table[ca].astype(np.float32); b = table[cb].astype(np.float32).T
    z = rng.integers(-4, 5, size=(M, N)).astype(np.float32)
    ta = torch.from_numpy(ca).to(gpu).view(tdt)
    tb = torch.from_numpy(cb).to(gpu).view(tdt).t()
    for add_dt in ("fp32", "bf16"):
        tz = from_np(z, add_dt, gpu)
        for add_np, add_t in ((z, tz), (z[:, :1], tz[:, :1]), (z[:1, :], tz[:1, :])):
            got = to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32, add=add_t))
            assert bits_equal(got, gemm.dot_epilogue(a, b, add=add_np)), (fmt, add_dt, add_np.shape)


@pytest.mark.parametrize("tile", [None, 0, 1, 2, 3, 4, 5, 6, 7])
def test_row_major_fp8_b_under_every_tile_choice_with_addend_activation_and_fp8_output(gpu, monkeypatch, tile):
    # whatever kernel the tuning knob asks for, a row-major fp8 B ends on a kernel that has the layout (the four-wave
    # one for 6, the 128x128 tiles for 1, the 256x256 one-barrier-per-step tiles otherwise); epilogues with an addend,
    # leaky_relu and an fp8 result go through the tile kernels' general epilogue.  Integer data: exact, and bit-equal
    # to the K-major call of the same product.
    if tile is not None:
        set_knob(monkeypatch, "MI355_GEMM_TILE", tile)
    M, N, K = 512, 768, 512
    rng = np.random.default_rng(3 if tile is None else tile)
    a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    b = rng.integers(-3, 4, size=(K, N)).astype(np.float32)
    z = rng.integers(-4, 5, size=(M, N)).astype(np.float32)
    ta = torch.from_numpy(formats.encode_fp8(a, "e4m3")).to(gpu).view(torch.float8_e4m3fn)
    tb = torch.from_numpy(formats.encode_fp8(b, "e4m3")).to(gpu).view(torch.float8_e4m3fn)     # [K, N] row-major
    tbk = tb.t().contiguous().t()
    tz = torch.from_numpy(z).to(gpu)
    assert np.array_equal(to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32)), a.astype(np.float64) @ b.astype(np.float64))
    got = triton_amd.matmul(ta, tb, out_dtype=torch.float32, add=tz, activation="leaky_relu")
    assert bits_equal(to_np(got), gemm.dot_epilogue(a, b, add=z, activation="leaky_relu"))
    assert torch.equal(got, triton_amd.matmul(ta, tbk, out_dtype=torch.float32, add=tz, activation="leaky_relu"))
    out8 = triton_amd.matmul(ta, tb, out_dtype=torch.float8_e4m3fn, a_scale=0.125)
    assert torch.equal(out8.view(torch.uint8), triton_amd.matmul(ta, tbk, out_dtype=torch.float8_e4m3fn, a_scale=0.125).view(torch.uint8))
    assert np.array_equal(out8.view(torch.uint8).cpu().numpy(), formats.encode_fp8((a @ b) * 0.125, "e4m3"))


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("shape", [(64, 64, 64), (128, 128, 64), (512, 768, 256), (300, 200, 136), (100, 70, 50), (16, 256, 512),
                                   (1024, 32, 256), (100, 2048, 64), (2048, 128, 64)])
def test_fused_epilogues_of_the_reference_dot_test(gpu, dtype, shape):
    # add-matrix / add-rows / add-cols / softmax / chain-dot (python/test/unit/language/test_core.py:3128-3145)
    # through mi355_gemm_epilogue: MFMA tile kernels, the any-stride kernel (100, 70, 50) and four skinny
    # shapes (the streaming kernels add the addend in their own epilogue; the second one runs with the
    # operands swapped, the last two as two launches of 64 rows and the rest).  Integer data: bit-exact.
    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
    z = rng.integers(-4, 5, size=(M, N)).astype(np.float32)
    ta, tb = from_np(a, dtype, gpu), from_np(b, dtype, gpu)
    for add_dt in ("fp32", dtype):
        tz = from_np(z, add_dt, gpu)
        for add_np, add_t in ((z, tz), (z[:, :1], tz[:, :1]), (z[:1, :], tz[:1, :]), (z[0], tz[0])):
            got = to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32, add=add_t))
            assert bits_equal(got, gemm.dot_epilogue(a, b, add=add_np)), (dtype, shape, add_dt, add_np.shape)
    # in place: C holds the addend and receives the result (the reference adds to the old Z)
    from triton_amd import _lib
    tc = from_np(z, "fp32", gpu)
    rc = _lib.load().mi355_gemm_epilogue(ta.data_ptr(), tb.data_ptr(), tc.data_ptr(), M, N, K, K, 1, N, 1, N, 1,
                                         _lib.BF16 if dtype == "bf16" else _lib.F16, _lib.F32, 0, 0,
                                         tc.data_ptr(), N, 1, _lib.F32, _lib.ACT_LEAKY_RELU, 0,
                                         torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert np.allclose(to_np(tc), gemm.dot_epilogue(a, b, add=z, activation="leaky_relu"), rtol=1e-6, atol=0)
    # softmax on small-magnitude data, output in the input type and in fp32
    a2, b2 = randn_rounded(rng, (M, K), dtype, 0.3), randn_rounded(rng, (K, N), dtype, 0.3)
    ta2, tb2 = from_np(a2, dtype, gpu), from_np(b2, dtype, gpu)
    bias = randn_rounded(rng, (1, N), "fp32")
    got = to_np(triton_amd.matmul(ta2, tb2, out_dtype=torch.float32, add=from_np(bias, "fp32", gpu), softmax=True))
    ref = gemm.dot_epilogue(a2, b2, add=bias, softmax=True)
    assert np.allclose(got, ref, rtol=1e-2, atol=1e-3) and np.allclose(got.sum(axis=1), 1.0, atol=1e-4)
    # 16-bit output: probabilities are about 1 / N, so the comparison is RELATIVE.  Rows of at most 256 columns are
    # normalised inside the tile on the fp32 accumulator (one rounding, like the oracle); wider rows by a second
    # launch that re-reads the rounded logits (two roundings: a looser bound)
    got16 = to_np(triton_amd.matmul(ta2, tb2, softmax=True))
    ref16 = gemm.dot_epilogue(a2, b2, softmax=True, out_dtype=dtype)
    assert np.allclose(got16, ref16, rtol=(1e-2 if N <= 256 else 6e-2), atol=1e-6), np.abs(got16 / ref16 - 1).max()
    # larger logits (|z| up to ~10): fused path only
    if N <= 256:
        a3, b3 = randn_rounded(rng, (M, K), dtype, 1.0), randn_rounded(rng, (K, N), dtype, 1.0)
        got3 = to_np(triton_amd.matmul(from_np(a3, dtype, gpu), from_np(b3, dtype, gpu), softmax=True, out_dtype=torch.float32))
        ref3 = gemm.dot_epilogue(a3, b3, softmax=True)
        assert np.allclose(got3, ref3, rtol=1e-2, atol=1e-7) and np.allclose(got3.sum(axis=1), 1.0, atol=1e-4)
    # chain-dot: (A @ B) rounded to the input type, then @ W
    w = rng.integers(-2, 3, size=(N, N)).astype(np.float32)
    got = to_np(triton_amd.chain_dot(ta, tb, from_np(w, dtype, gpu), out_dtype=torch.float32))
    assert bits_equal(got, gemm.dot_epilogue(a, b, chain_w=w, mid_dtype=dtype))
    wr = randn_rounded(rng, (N, N), dtype, 0.3)
    got = to_np(triton_amd.chain_dot(ta2, tb2, from_np(wr, dtype, gpu)))
    assert np.allclose(got, gemm.dot_epilogue(a2, b2, chain_w=wr, mid_dtype=dtype, out_dtype=dtype), rtol=1e-2, atol=1e-2)
    # a non-square W, K-major B, addend + softmax in front of the chained product
    n2 = 72 if N <= 256 else 320
    w2 = rng.integers(-2, 3, size=(N, n2)).astype(np.float32)
    tbk = tb.t().contiguous().t()
    got = to_np(triton_amd.chain_dot(ta, tbk, from_np(w2, dtype, gpu), out_dtype=torch.float32, add=from_np(z[:, :1], "fp32", gpu)))
    assert bits_equal(got, gemm.dot_epilogue(a, b, add=z[:, :1], chain_w=w2, mid_dtype=dtype))
    got = to_np(triton_amd.chain_dot(ta2, tb2, from_np(w2, dtype, gpu), out_dtype=torch.float32, softmax=True))
    ref = gemm.dot_epilogue(a2, b2, softmax=True, chain_w=w2, mid_dtype=dtype)
    # (one launch: z rounded once; the two-launch fall-back for wide rows rounds the logits, then the probabilities)
    assert np.allclose(got, ref, rtol=2e-2, atol=2e-3 if N <= 256 else 3e-2), np.abs(got - ref).max()


def test_skinny_16bit_full_decode_size(gpu):
    # the table's largest decode shape, M = 16, N = K = 8192 fp16 with a row-major B, against the
    # fp64 closed form; plus linearity in A (exact: the second operand doubles every product)
    rng = np.random.default_rng(31)
    a = randn_rounded(rng, (16, 8192), "fp16", 0.25)
    b = randn_rounded(rng, (8192, 8192), "fp16", 0.25)
    ta, tb = from_np(a, "fp16", gpu), from_np(b, "fp16", gpu)
    c = to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32))
    assert np.allclose(c, gemm.matmul_closed_form(a, b), rtol=1e-2, atol=1e-2)
    c2 = to_np(triton_amd.matmul(ta * 2, tb, out_dtype=torch.float32))
    assert bits_equal(c2, 2 * c)
    # the same product with the weight stored K-contiguous (x @ W^T, the whole-line form of the streaming kernel) and
    # with 64 rows of A (X in whole lines too): the same sums in another order, so equal to the tolerance - and exact
    # on the integer operands of the second pair
    tbk = tb.t().contiguous().t()
    ck = to_np(triton_amd.matmul(ta, tbk, out_dtype=torch.float32))
    assert np.allclose(ck, c, rtol=1e-3, atol=1e-3)
    ai = rng.integers(-2, 3, size=(64, 8192)).astype(np.float32)
    bi = rng.integers(-2, 3, size=(8192, 8192)).astype(np.float32)
    tai, tbi = from_np(ai, "fp16", gpu), from_np(bi, "fp16", gpu)
    want = gemm.matmul_closed_form(ai, bi, out_dtype="fp32")
    assert bits_equal(to_np(triton_amd.matmul(tai, tbi, out_dtype=torch.float32)), want)
    assert bits_equal(to_np(triton_amd.matmul(tai, tbi.t().contiguous().t(), out_dtype=torch.float32)), want)


@pytest.mark.parametrize("nprog", [None, 7, 3])
@pytest.mark.parametrize("dtype", ["fp16", "bf16", "e4m3"])
def test_stream_k_schedule_is_bit_exact_on_integers(gpu, monkeypatch, dtype, nprog):
    # mi355_gemm_streamk: programs split all K steps of all 256x256 tiles evenly.  With the device's
    # CU count (None) these small products are split-K (more programs than tiles); with 7 or 3
    # programs ranges begin and end inside tiles and span whole tiles in between.  Integer data: the
    # partial sums are exact, so any split gives the bits of the closed form.  Shapes the schedule
    # does not take (partial tiles, K tails) run as plain calls.
    if nprog is not None:
        set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", str(nprog))
    rng = np.random.default_rng(17 + (nprog or 0))
    for (M, N, K) in [(512, 768, 1024), (256, 256, 4096), (1280, 256, 512), (300, 264, 520), (16, 512, 256)]:
        a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
        ref = gemm.matmul_closed_form(a, b, out_dtype="fp32")
        if dtype == "e4m3":
            ca, cb = formats.encode_fp8(a, "e4m3"), formats.encode_fp8(np.ascontiguousarray(b.T), "e4m3")
            ta = torch.from_numpy(ca).to(gpu).view(torch.float8_e4m3fn)
            tbs = [torch.from_numpy(cb).to(gpu).view(torch.float8_e4m3fn).t()]
        else:
            ta = from_np(a, dtype, gpu)
            tbs = [from_np(b, dtype, gpu), from_np(np.ascontiguousarray(b.T), dtype, gpu).t()]
        for tb in tbs:
            got = to_np(triton_amd.matmul_streamk(ta, tb, out_dtype=torch.float32))
            assert bits_equal(got, ref), (dtype, nprog, M, N, K, tb.stride())
    # random data against the closed form, output in the input type
    if dtype != "e4m3":
        a2, b2 = randn_rounded(rng, (768, 1024), dtype), randn_rounded(rng, (1024, 512), dtype)
        c = to_np(triton_amd.matmul_streamk(from_np(a2, dtype, gpu), from_np(b2, dtype, gpu)))
        assert np.allclose(c, gemm.matmul_closed_form(a2, b2, out_dtype=dtype), rtol=1e-2, atol=1e-2)


def test_lean_and_general_epilogue_of_the_four_wave_kernels_agree_bit_for_bit(gpu, monkeypatch):
    # the four-wave kernels have a lean epilogue (16-bit C with unit column stride, per-tensor scales, nothing else)
    # as instantiations of their own; MI355_GEMM_LEAN_EPILOGUE=0 sends the same products through the general one
    rng = np.random.default_rng(77)
    M = N = 2560
    K = 1024
    a16, b16 = (randn_rounded(rng, s, "bf16", 1.0) for s in ((M, K), (K, N)))
    ta, tb = from_np(a16, "bf16", gpu), from_np(b16, "bf16", gpu)
    q = lambda shape: torch.from_numpy(rng.integers(0, 0x78, size=shape).astype(np.uint8)).to(gpu).view(torch.float8_e4m3fn)
    qa, qb = q((M, K)), q((N, K))
    pa, pb = (torch.from_numpy(rng.integers(0, 256, size=(M, K // 2)).astype(np.uint8)).to(gpu) for _ in range(2))
    sa, sb = (torch.from_numpy(rng.integers(123, 132, size=(M, K // 32)).astype(np.uint8)).to(gpu) for _ in range(2))
    cases = {
        "bf16": lambda: triton_amd.matmul(ta, tb),
        "bf16 K-major B, K tail": lambda: triton_amd.matmul(ta[:, :K - 8].contiguous(), tb.t().contiguous().t()[:K - 8]),
        "fp8 scaled -> bf16": lambda: triton_amd.matmul(qa, qb.t(), a_scale=0.37, b_scale=1.9, out_dtype=torch.bfloat16),
        "fp8 scaled -> fp16": lambda: triton_amd.matmul(qa, qb.t(), a_scale=0.01, b_scale=0.02, out_dtype=torch.float16),
        "mxfp4 -> bf16": lambda: triton_amd.mx_matmul(pa, sa, pb, sb, "mxfp4", out_dtype=torch.bfloat16),
        "mxfp8 -> fp16": lambda: triton_amd.mx_matmul(pa.repeat(1, 2) & 0x77, sa, pb.repeat(1, 2) & 0x77, sb, "mxfp8", out_dtype=torch.float16),
    }
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    results = {}
    for lean in ("1", "0"):
        set_knob(monkeypatch, "MI355_GEMM_LEAN_EPILOGUE", lean)
        for name, fn in cases.items():
            if lean == "0" and "K tail" in name:
                continue        # (the tail form exists with the lean epilogue only; without it another kernel runs)
            results[name, lean] = to_np(fn())
    for name in cases:
        if "K tail" in name:
            ref = a16[:, :K - 8].astype(np.float64) @ b16[:K - 8].astype(np.float64)
            assert np.allclose(results[name, "1"], ref, atol=1e-2 * np.abs(ref).max(), rtol=1e-2), name
        else:
            assert bits_equal(results[name, "1"], results[name, "0"]), name


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("N", [1004, 1001])
def test_n_not_a_multiple_of_16_bytes_takes_the_fast_kernels_through_a_padded_pitch(gpu, dtype, N):
    # rows of a row-major B that do not start on 16-byte boundaries cannot be loaded by the MFMA kernels; the wrapper
    # copies such a B into rows of a padded pitch instead of leaving the product to the any-stride kernel.
    # Integer-valued operands: exact sums, so the result is that kernel's bit for bit, in a C of the caller's shape.
    rng = np.random.default_rng(N)
    M, K = 1024, 1536       # (large enough for the wrapper to copy: 2^30 multiply-adds)
    ai = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    bi = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
    got = triton_amd.matmul(from_np(ai, dtype, gpu), from_np(bi, dtype, gpu), out_dtype=torch.float32)
    assert got.shape == (M, N) and got.is_contiguous()
    assert bits_equal(to_np(got), (ai.astype(np.float64) @ bi.astype(np.float64)).astype(np.float32))
    a, b = randn_rounded(rng, (M, K), dtype, 1.0), randn_rounded(rng, (K, N), dtype, 1.0)
    got = to_np(triton_amd.matmul(from_np(a, dtype, gpu), from_np(b, dtype, gpu)))
    ref = a.astype(np.float64) @ b.astype(np.float64)
    assert np.allclose(got, ref, rtol=1e-2, atol=1e-2 * np.abs(ref).max())
    # a B that already lives in a buffer with a padded pitch (rows start on 16-byte boundaries, N is no multiple) is
    # taken as it is: the last chunk of a row reaches into the padding - filled with NaN here, which must not show
    wide = torch.full((K, N + 16 - N % 8), float("nan"), dtype=torch.float32, device=gpu).to(from_np(bi, dtype, gpu).dtype)
    wide[:, :N] = from_np(bi, dtype, gpu)
    got = triton_amd.matmul(from_np(ai, dtype, gpu), wide[:, :N], out_dtype=torch.float32)
    assert bits_equal(to_np(got), (ai.astype(np.float64) @ bi.astype(np.float64)).astype(np.float32))


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5])
def test_padded_pitch_row_major_b_under_every_tile_kernel(gpu, monkeypatch, tile):
    # N = 2052 in rows of 2056 elements (NaN in the padding), enough tiles for the large-product kernels: every tile
    # kernel clamps its last chunk of a B row to N rounded up to whole chunks.  Integer data: exact.
    set_knob(monkeypatch, "MI355_GEMM_TILE", tile)
    rng = np.random.default_rng(50 + tile)
    M, N, K = 1024, 2052, 320
    a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
    ref = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    for dtype in ("bf16", "fp16"):
        wide = torch.full((K, N + 4), float("nan"), dtype=torch.float32, device=gpu).to(from_np(b, dtype, gpu).dtype)
        wide[:, :N] = from_np(b, dtype, gpu)
        got = triton_amd.matmul(from_np(a, dtype, gpu), wide[:, :N], out_dtype=torch.float32)
        assert bits_equal(to_np(got), ref), (tile, dtype)


@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_row_major_fp8_b_with_n_not_a_multiple_of_16_in_a_padded_pitch(gpu, fmt, tdt):
    # the fp8 case of the same: N = 1000 in rows of 1008 bytes, and through the wrapper's padding copy (pitch 1000)
    rng = np.random.default_rng(41)
    M, N, K = 1024, 1000, 1536
    a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    b = rng.integers(-3, 4, size=(K, N)).astype(np.float32)
    ta = torch.from_numpy(formats.encode_fp8(a, fmt)).to(gpu).view(tdt)
    tb = torch.from_numpy(formats.encode_fp8(b, fmt)).to(gpu).view(tdt)
    ref = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    wide = torch.full((K, 1008), 0x7f if fmt == "e4m3" else 0x7e, dtype=torch.uint8, device=gpu)    # NaN codes
    wide[:, :N] = tb.view(torch.uint8)
    for bb in (tb, wide.view(tdt)[:, :N]):
        got = triton_amd.matmul(ta, bb, out_dtype=torch.float32)
        assert got.shape == (M, N) and bits_equal(to_np(got), ref), bb.stride()


@pytest.mark.parametrize("case", ["bf16 row-major B", "fp16 K-major B", "fp8"])
def test_k_not_a_multiple_of_16_bytes_takes_the_fast_kernels_through_zero_padding(gpu, case):
    # rows that are not 16-byte multiples cannot be loaded by the MFMA kernels; the wrapper appends the zeros that the
    # reference's K-tail mask stands for (03:297-298) instead of leaving the product to the strided kernel
    rng = np.random.default_rng(5)
    M, N = 512, 768
    if case == "fp8":
        K = 4104      # a multiple of 8 but not of 16 bytes
        a = rng.integers(0, 0x78, size=(M, K)).astype(np.uint8)
        b = rng.integers(0, 0x78, size=(N, K)).astype(np.uint8)
        ta = torch.from_numpy(a).to(gpu).view(torch.float8_e4m3fn)
        tb = torch.from_numpy(b).to(gpu).view(torch.float8_e4m3fn).t()
        got = to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32))
        ref = ta.float().cpu().numpy().astype(np.float64) @ tb.float().cpu().numpy().astype(np.float64)
        assert np.allclose(got, ref, rtol=3e-2, atol=3e-2 * np.abs(ref).max())
        return
    K = 4100
    dtype = "bf16" if case.startswith("bf16") else "fp16"
    a, b = randn_rounded(rng, (M, K), dtype, 1.0), randn_rounded(rng, (K, N), dtype, 1.0)
    ta, tb = from_np(a, dtype, gpu), from_np(b, dtype, gpu)
    if "K-major" in case:
        tb = tb.t().contiguous().t()
    got = to_np(triton_amd.matmul(ta, tb))
    ref = a.astype(np.float64) @ b.astype(np.float64)
    assert got.shape == (M, N)
    assert np.allclose(got, ref, rtol=1e-2, atol=1e-2 * np.abs(ref).max())
    # integer-valued operands: exact sums, so the padded product is the strided kernel's product bit for bit
    ai = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    bi = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
    exact = to_np(triton_amd.matmul(from_np(ai, dtype, gpu), from_np(bi, dtype, gpu), out_dtype=torch.float32))
    assert bits_equal(exact, (ai.astype(np.float64) @ bi.astype(np.float64)).astype(np.float32))


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("kmajor", [False, True])
@pytest.mark.parametrize("shape", [(192, 256, 256), (1536, 1024, 1280), (3072, 768, 512)])
def test_four_wave_kernel_on_tiles_of_192_rows_is_bit_exact(gpu, monkeypatch, dtype, kmajor, shape):
    # M a multiple of 192: the four-wave kernel also runs on tiles of 192 x 256 (chosen by itself where they fill
    # the CUs better, forced here); small integers make every sum exact
    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
    ta, tb = from_np(a, dtype, gpu), from_np(b, dtype, gpu)
    if kmajor:
        tb = tb.t().contiguous().t()
    ref = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    set_knob(monkeypatch, "MI355_GEMM_TILE_M", "192")
    got = to_np(triton_amd.matmul(ta, tb))
    assert bits_equal(got, to_np(from_np(ref, dtype, gpu))), "tiles of 192 rows"
    set_knob(monkeypatch, "MI355_GEMM_TILE_M", "128")
    assert bits_equal(to_np(triton_amd.matmul(ta, tb)), got), "tiles of 128 rows"
    set_knob(monkeypatch, "MI355_GEMM_TILE_M", "256")
    assert bits_equal(to_np(triton_amd.matmul(ta, tb)), got), "tiles of 256 rows"


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("kmajor", [False, True])
@pytest.mark.parametrize("programs", [3, 256])
def test_two_tile_heights_in_one_launch_are_bit_exact(gpu, monkeypatch, dtype, kmajor, programs):
    # the upper rows of C on 256-row tiles and the lower ones on 192-row tiles, one launch (chosen by itself for tile
    # counts that fill the last round of CUs badly, forced here): one tile of each kind, several of each per program,
    # more programs than tiles of either kind.  Small integers make every sum exact.
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", programs)
    for (rows256, M, N, K) in [(256, 448, 256, 256), (256, 1216, 512, 512), (1280, 2240, 768, 1280), (768, 960, 1024, 384)]:
        rng = np.random.default_rng(M + N + K + programs)
        a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
        ta, tb = from_np(a, dtype, gpu), from_np(b, dtype, gpu)
        if kmajor:
            tb = tb.t().contiguous().t()
        ref = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
        set_knob(monkeypatch, "MI355_GEMM_MIXED_ROWS", rows256)
        got = to_np(triton_amd.matmul(ta, tb))
        assert bits_equal(got, to_np(from_np(ref, dtype, gpu))), (rows256, M, N, K)
        set_knob(monkeypatch, "MI355_GEMM_MIXED_ROWS", 0)
        assert bits_equal(to_np(triton_amd.matmul(ta, tb)), got)


@pytest.mark.parametrize("programs", [3, 256])
@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_two_tile_heights_in_one_launch_are_bit_exact_for_fp8(gpu, monkeypatch, fmt, tdt, programs):
    # the fp8 form of the same launch (K-major B, 16-bit C)
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", programs)
    for (rows256, M, N, K) in [(256, 448, 256, 256), (256, 1216, 512, 1024), (1280, 2240, 768, 1280), (768, 960, 1024, 512)]:
        rng = np.random.default_rng(M + N + K + programs + len(fmt))
        a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
        b = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
        ta = torch.from_numpy(formats.encode_fp8(a, fmt)).to(gpu).view(tdt)
        tb = torch.from_numpy(formats.encode_fp8(b, fmt)).to(gpu).view(tdt).t()
        for out, name in ((torch.bfloat16, "bf16"), (torch.float16, "fp16")):
            set_knob(monkeypatch, "MI355_GEMM_MIXED_ROWS", rows256)
            got = to_np(triton_amd.matmul(ta, tb, out_dtype=out))
            assert bits_equal(got, gemm.matmul_closed_form(a, b.T, out_dtype=name)), (rows256, M, N, K, fmt, programs, name)
            set_knob(monkeypatch, "MI355_GEMM_MIXED_ROWS", 0)
            assert bits_equal(to_np(triton_amd.matmul(ta, tb, out_dtype=out)), got)


def test_5120_cubed_takes_two_tile_heights_and_matches_sampled_rows(gpu):
    # 400 tiles of 256 x 256 for 256 CUs: the size heuristic splits M into 2816 rows of 256-row and 2304 of 192-row tiles
    rng = np.random.default_rng(12)
    n = 5120
    a, b = randn_rounded(rng, (n, n), "bf16", 1.0), randn_rounded(rng, (n, n), "bf16", 1.0)
    got = to_np(triton_amd.matmul(from_np(a, "bf16", gpu), from_np(b, "bf16", gpu)))
    rows = np.concatenate([rng.choice(n, size=20, replace=False), [0, 2815, 2816, 3007, 3008, n - 1]])
    ref = a[rows].astype(np.float64) @ b.astype(np.float64)
    assert np.allclose(got[rows], ref, rtol=1e-2, atol=1e-2 * np.abs(ref).max())


@pytest.mark.parametrize("programs", [3, 256])
@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_four_wave_fp8_kernel_on_tiles_of_192_rows_is_bit_exact(gpu, monkeypatch, fmt, tdt, programs):
    # the fp8 form of the same tiles (K-major B, 16-bit C): six A fragments per wave, 14 loads per K step (128 rows:
    # four and 12); one and several tiles per program.  Integer data: the bits of the exact product, and of the
    # 256-row tiles' result.
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", programs)
    rng = np.random.default_rng(programs + len(fmt))
    for (M, N, K) in [(192, 256, 256), (1536, 1024, 1280), (3072, 768, 512), (576, 512, 2048), (384, 256, 768)]:
        a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
        b = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
        ta = torch.from_numpy(formats.encode_fp8(a, fmt)).to(gpu).view(tdt)
        tb = torch.from_numpy(formats.encode_fp8(b, fmt)).to(gpu).view(tdt).t()
        for out, name in ((torch.bfloat16, "bf16"), (torch.float16, "fp16")):
            set_knob(monkeypatch, "MI355_GEMM_TILE_M", "192")
            got = to_np(triton_amd.matmul(ta, tb, out_dtype=out))
            assert bits_equal(got, gemm.matmul_closed_form(a, b.T, out_dtype=name)), (M, N, K, fmt, programs, name)
            set_knob(monkeypatch, "MI355_GEMM_TILE_M", "256")
            assert bits_equal(to_np(triton_amd.matmul(ta, tb, out_dtype=out)), got)
            if M % 128 == 0:
                set_knob(monkeypatch, "MI355_GEMM_TILE_M", "128")
                assert bits_equal(to_np(triton_amd.matmul(ta, tb, out_dtype=out)), got), "tiles of 128 rows"


def test_3072_cubed_takes_the_192_row_tiles_and_matches_sampled_rows(gpu):
    # 144 tiles of 256 x 256 for 256 CUs, 192 tiles of 192 x 256: the size heuristic picks the latter
    rng = np.random.default_rng(11)
    n = 3072
    a, b = randn_rounded(rng, (n, n), "bf16", 1.0), randn_rounded(rng, (n, n), "bf16", 1.0)
    got = to_np(triton_amd.matmul(from_np(a, "bf16", gpu), from_np(b, "bf16", gpu)))
    rows = rng.choice(n, size=24, replace=False)
    ref = a[rows].astype(np.float64) @ b.astype(np.float64)
    assert np.allclose(got[rows], ref, rtol=1e-2, atol=1e-2 * np.abs(ref).max())


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(512, 512, 512), (4096, 4096, 512)])
@pytest.mark.parametrize("pad", [4, 8])
def test_c_rows_of_8_and_16_byte_alignment_through_the_c_abi(gpu, shape, pad):
    # The short epilogues store 16 bytes per lane (neighbouring accumulator groups exchanged between lanes first),
    # which needs C rows of 16-byte alignment; a row pitch that is a multiple of 4 but not of 8 elements takes the
    # general epilogue with its 8-byte stores.  Both through mi355_gemm directly with C a view into a wider buffer
    # (the Python surface always allocates a dense C): small tiles and the four-wave kernel, integer data, the bits
    # of the closed form, and the columns beyond N untouched.
    from triton_amd import _lib

    M, N, K = shape
    rng = np.random.default_rng(M + pad)
    a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
    ta, tb = from_np(a, "bf16", gpu), from_np(b, "bf16", gpu)
    buf = torch.full((M, N + pad), 7.0, dtype=torch.bfloat16, device=gpu)
    c = buf[:, :N]
    rc = _lib.load().mi355_gemm(ta.data_ptr(), tb.data_ptr(), c.data_ptr(), M, N, K,
                                ta.stride(0), ta.stride(1), tb.stride(0), tb.stride(1), c.stride(0), c.stride(1),
                                _lib.BF16, _lib.BF16, None, None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert bits_equal(to_np(c), gemm.matmul_closed_form(a, b, out_dtype="bf16")), (shape, pad)
    assert bool((buf[:, N:] == 7.0).all())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("shape", [(16, 16384, 512), (7, 32768, 192), (32, 16448, 96), (1, 16384, 2048)])
def test_skinny_kernel_with_64_columns_per_workgroup_is_bit_exact(gpu, dtype, shape):
    # a row-major B wide enough that 64 columns per workgroup still cover the compute units (N / 64 >= 256): the
    # form of the streaming kernel that fetches whole 128-byte lines of B - two column tiles per wave, eight waves
    # splitting K, k rows with bit 1 set stored with their halves swapped.  Exact integer sums (K from 3 to 64
    # stages, so some waves get none), every M class, an epilogue with the addend; N = 16448 has 257 workgroups.
    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
    d = rng.integers(-3, 4, size=(M, N)).astype(np.float32)
    ta, tb, td = from_np(a, dtype, gpu), from_np(b, dtype, gpu), torch.from_numpy(d).to(gpu)
    got = to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32))
    assert bits_equal(got, gemm.matmul_closed_form(a, b, out_dtype="fp32")), (dtype, shape)
    got = to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32, add=td))
    assert bits_equal(got, gemm.matmul_closed_form(a, b, out_dtype="fp32") + d), (dtype, shape, "addend")


@pytest.mark.parametrize("dtype", ["fp16", "bf16", "e4m3", "fp32"])
@pytest.mark.parametrize("splits", [0, 2, 3, 7, 32])
def test_split_k_is_bit_exact_on_integers(gpu, dtype, splits):
    # mi355_gemm_splitk through the C ABI: `splits` workgroups per 128x128 tile, fp32 partial tiles in the workspace,
    # a second launch adds them in split order and does the epilogue.  Integer data: every partial sum is exact, so
    # any split gives the bits of the closed form.  Shapes: partial tiles on both sides, a K that is not a multiple
    # of the split, a K with a tail below one 64-byte step, one tile only; both layouts of B; a strided C.
    lib = _lib.load()
    rng = np.random.default_rng(23 + splits)
    abi = {"fp16": _lib.F16, "bf16": _lib.BF16, "e4m3": _lib.F8E4M3, "fp32": _lib.F32}[dtype]
    for (M, N, K) in [(256, 256, 4096), (130, 96, 8192), (384, 200, 2096), (128, 128, 16384), (512, 640, 1056)]:
        a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
        ref = gemm.matmul_closed_form(a, b, out_dtype="fp32")
        if dtype == "e4m3":
            ta = torch.from_numpy(formats.encode_fp8(a, "e4m3")).to(gpu).view(torch.float8_e4m3fn)
            tbs = [torch.from_numpy(formats.encode_fp8(np.ascontiguousarray(b.T), "e4m3")).to(gpu).view(torch.float8_e4m3fn).t()]
            if N % 16 == 0:
                tbs.append(torch.from_numpy(formats.encode_fp8(b, "e4m3")).to(gpu).view(torch.float8_e4m3fn))
        else:
            ta = from_np(a, dtype, gpu)
            tbs = [from_np(np.ascontiguousarray(b.T), dtype, gpu).t()]
            if N % 8 == 0:
                tbs.append(from_np(b, dtype, gpu))     # (fp32: no tile kernel for a row-major B - the plain call's any-stride kernel)
        ws = torch.full((32 * M * N,), float("nan"), dtype=torch.float32, device=gpu)   # (contents must not matter)
        for tb in tbs:
            cbuf = torch.full((M, N + 5), 7.0, dtype=torch.float32, device=gpu)
            c = cbuf[:, :N]
            rc = lib.mi355_gemm_splitk(ta.data_ptr(), tb.data_ptr(), c.data_ptr(), M, N, K, ta.stride(0), ta.stride(1),
                                       tb.stride(0), tb.stride(1), c.stride(0), c.stride(1), abi, _lib.F32, None, None,
                                       _lib.ACT_NONE, splits, ws.data_ptr(), ws.numel() * 4, torch.cuda.current_stream().cuda_stream)
            assert rc == 0, (rc, dtype, splits, M, N, K)
            assert bits_equal(to_np(c), ref), (dtype, splits, M, N, K, tb.stride())
            assert bool((cbuf[:, N:] == 7.0).all())


def test_split_k_epilogue_and_the_route_from_matmul(gpu, monkeypatch):
    # the epilogue of the second launch (scales, leaky_relu, one rounding to the output type) against the closed form,
    # and matmul() itself: with the split switched off it must give the same bits on integers and agree to 1e-2 on
    # random data; a workspace that is too small is refused before any launch
    lib = _lib.load()
    rng = np.random.default_rng(5)
    M, N, K = 256, 384, 8192
    a, b = randn_rounded(rng, (M, K), "bf16"), randn_rounded(rng, (K, N), "bf16")
    ta, tb = from_np(a, "bf16", gpu), from_np(b, "bf16", gpu)
    ref = gemm.matmul_closed_form(a, b, out_dtype="bf16", activation="leaky_relu")
    got = to_np(triton_amd.matmul(ta, tb, activation="leaky_relu"))
    assert np.allclose(got, ref, rtol=1e-2, atol=1e-2)
    set_knob(monkeypatch, "MI355_GEMM_SPLITK", "0")
    plain = to_np(triton_amd.matmul(ta, tb, activation="leaky_relu"))
    assert np.allclose(plain, ref, rtol=1e-2, atol=1e-2)
    monkeypatch.delenv("MI355_GEMM_SPLITK")
    ai = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    bi = rng.integers(-3, 4, size=(K, N)).astype(np.float32)
    tai, tbi = from_np(ai, "fp16", gpu), from_np(bi, "fp16", gpu)
    refi = gemm.matmul_closed_form(ai, bi, out_dtype="fp32")
    assert bits_equal(to_np(triton_amd.matmul(tai, tbi, out_dtype=torch.float32)), refi)
    # fp8 with per-tensor scales and an fp8 output: the scales multiply the sum of the slices once
    qa = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    qb = rng.integers(-2, 3, size=(N, K)).astype(np.float32)
    tqa = torch.from_numpy(formats.encode_fp8(qa, "e4m3")).to(gpu).view(torch.float8_e4m3fn)
    tqb = torch.from_numpy(formats.encode_fp8(qb, "e4m3")).to(gpu).view(torch.float8_e4m3fn)
    got8 = to_np(triton_amd.matmul(tqa, tqb.t(), a_scale=0.5, b_scale=0.25, out_dtype=torch.bfloat16))
    assert bits_equal(got8, formats.round_to((qa @ qb.T) * 0.125, "bf16"))
    c = torch.empty((M, N), dtype=torch.bfloat16, device=gpu)
    ws = torch.empty(M * N, dtype=torch.float32, device=gpu)
    rc = lib.mi355_gemm_splitk(ta.data_ptr(), tb.data_ptr(), c.data_ptr(), M, N, K, K, 1, N, 1, N, 1, _lib.BF16, _lib.BF16,
                               None, None, _lib.ACT_NONE, 4, ws.data_ptr(), ws.numel() * 4, torch.cuda.current_stream().cuda_stream)
    assert rc == -1   # MI355_EINVAL


@pytest.mark.parametrize("dtype", ["fp16", "bf16", "e4m3", "fp32"])
def test_random_shapes_through_the_default_dispatch_are_bit_exact(gpu, dtype):
    # Whatever kernel the size heuristics pick - four-wave tiles of three heights, two heights in one launch, 128x128
    # tiles, split-K, skinny, masked, padded pitches - the product of small integers has exactly representable partial
    # sums, so the result must be the closed form's bits (rounded once where the output is 16-bit).  Seeded shapes
    # around the heuristics' thresholds: multiples of 64 .. 256 with and without a ragged remainder, both B layouts.
    rng = np.random.default_rng({"fp16": 101, "bf16": 202, "e4m3": 303, "fp32": 404}[dtype])
    base = [64, 128, 192, 256, 320, 384, 512, 640, 768, 1024, 1280, 1536, 2048, 2304, 2560, 3072]
    ks = [64, 128, 256, 320, 512, 1024, 1040, 2048, 4096, 8192]
    for case in range(26):
        M = int(rng.choice(base)) + int(rng.choice([0, 0, 0, 8, -8, 16, 1]))
        N = int(rng.choice(base)) + int(rng.choice([0, 0, 0, 8, -8, 16, 3]))
        K = int(rng.choice(ks)) + int(rng.choice([0, 0, 0, 8, 16, -16]))
        if M * N * K > 3072 * 3072 * 2048:   # (keeps the numpy reference to a fraction of a second per case)
            K = max(64, (3072 * 3072 * 2048 // (M * N)) // 64 * 64)
        kmajor = bool(rng.integers(0, 2))
        a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
        exact = a @ b                          # fp32 sums of integers below 2^24: exact in any order
        if dtype == "e4m3":
            ta = torch.from_numpy(formats.encode_fp8(a, "e4m3")).to(gpu).view(torch.float8_e4m3fn)
            if kmajor:
                tb = torch.from_numpy(formats.encode_fp8(np.ascontiguousarray(b.T), "e4m3")).to(gpu).view(torch.float8_e4m3fn).t()
            else:
                tb = torch.from_numpy(formats.encode_fp8(b, "e4m3")).to(gpu).view(torch.float8_e4m3fn)
            out = [torch.float32, torch.bfloat16, torch.float16][case % 3]
        else:
            ta = from_np(a, dtype, gpu)
            tb = from_np(np.ascontiguousarray(b.T), dtype, gpu).t() if kmajor else from_np(b, dtype, gpu)
            out = [torch.float32, None][case % 2]
        got = triton_amd.matmul(ta, tb) if out is None else triton_amd.matmul(ta, tb, out_dtype=out)
        name = {torch.float32: "fp32", torch.bfloat16: "bf16", torch.float16: "fp16", None: "fp16" if dtype == "fp32" else dtype}[out]
        assert bits_equal(to_np(got), formats.round_to(exact, name)), (dtype, case, M, N, K, kmajor, name)


@pytest.mark.parametrize("kmajor", [True, False])
def test_fp32_operands_are_multiplied_exactly(gpu, kmajor):
    # fp32 inputs: `tl.dot` of fp32 blocks accumulates exact fp32 products in fp32 (the interpreter's np.matmul in fp32,
    # python/triton/runtime/interpreter.py:542-549).  Integers beyond what any 16-bit type holds (|x| <= 3000, so a
    # detour through fp16 / bf16 would show) with sums that stay below 2^24: the result is the closed form's bits,
    # on the MFMA tiles (K-major B through the C ABI, a row-major B through the wrapper's transposing copy), on the
    # any-stride kernel (small products, K not a multiple of 4, a row-major B through the C ABI) and for every output
    # type; then N(0,1) data against the fp64 product at fp32 accuracy.
    lib = _lib.load()
    rng = np.random.default_rng(41 + kmajor)
    for (M, N, K) in [(256, 256, 64), (128, 128, 16), (300, 200, 72), (512, 384, 130), (2048, 2048, 256), (1024, 3072, 512), (64, 64, 4)]:
        a = rng.integers(-3000, 3001, size=(M, K)).astype(np.float32)
        b = rng.integers(-1, 2, size=(K, N)).astype(np.float32)
        ref = a.astype(np.float64) @ b.astype(np.float64)
        assert np.abs(ref).max() < 2 ** 24
        ta = torch.from_numpy(a).to(gpu)
        tb = torch.from_numpy(np.ascontiguousarray(b.T)).to(gpu).t() if kmajor else torch.from_numpy(b).to(gpu)
        got = triton_amd.matmul(ta, tb, out_dtype=torch.float32)
        assert bits_equal(to_np(got), ref.astype(np.float32)), (M, N, K, kmajor)
        # the C ABI itself, with the strides as they are
        c = torch.full((M, N + 3), 7.0, dtype=torch.float32, device=gpu)
        cv = c[:, :N]
        rc = lib.mi355_gemm(ta.data_ptr(), tb.data_ptr(), cv.data_ptr(), M, N, K, ta.stride(0), ta.stride(1), tb.stride(0), tb.stride(1),
                            cv.stride(0), cv.stride(1), _lib.F32, _lib.F32, None, None, _lib.ACT_NONE, torch.cuda.current_stream().cuda_stream)
        assert rc == 0 and bits_equal(to_np(cv), ref.astype(np.float32)) and bool((c[:, N:] == 7.0).all()), (M, N, K, kmajor)
    # the reference wrapper's own output type (03:338: fp16 whatever the inputs) and the activation
    a = rng.integers(-8, 9, size=(384, 96)).astype(np.float32)
    b = rng.integers(-8, 9, size=(96, 256)).astype(np.float32)
    ta, tb = torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu)
    got = triton_amd.matmul(ta, tb, activation="leaky_relu")
    assert got.dtype == torch.float16
    assert bits_equal(to_np(got), gemm.matmul_closed_form(a, b, activation="leaky_relu", out_dtype="fp16"))
    # random data: fp32 products and sums against fp64
    a = rng.normal(size=(1024, 2048)).astype(np.float32)
    b = rng.normal(size=(2048, 768)).astype(np.float32)
    ta = torch.from_numpy(a).to(gpu)
    tb = torch.from_numpy(np.ascontiguousarray(b.T)).to(gpu).t() if kmajor else torch.from_numpy(b).to(gpu)
    got = to_np(triton_amd.matmul(ta, tb, out_dtype=torch.float32))
    ref = a.astype(np.float64) @ b.astype(np.float64)
    err = report_error(f"fp32 1024 x 768 x 2048 kmajor={kmajor}", got, ref)
    assert err < 1e-5
    # every tile form of the fp32 kernel on whole and partial tiles, through mi355_gemm_tuned: the same bits on integers
    a = rng.integers(-300, 301, size=(768, 264)).astype(np.float32)
    b = rng.integers(-2, 3, size=(264, 520)).astype(np.float32)
    ta, tb = torch.from_numpy(a).to(gpu), torch.from_numpy(np.ascontiguousarray(b.T)).to(gpu).t()
    ref = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    for tile in (0, 1, 2, 3, 4, 5, 6):
        c = torch.empty(768, 520, dtype=torch.float32, device=gpu)
        rc = lib.mi355_gemm_tuned(ta.data_ptr(), tb.data_ptr(), c.data_ptr(), 768, 520, 264, 264, 1, 1, 264, 520, 1, _lib.F32, _lib.F32,
                                  None, None, _lib.ACT_NONE, tile, 8, torch.cuda.current_stream().cuda_stream)
        assert rc == 0 and bits_equal(to_np(c), ref), tile
    a = rng.integers(-300, 301, size=(512, 1024)).astype(np.float32)
    b = rng.integers(-2, 3, size=(1024, 768)).astype(np.float32)
    ta, tb = torch.from_numpy(a).to(gpu), torch.from_numpy(np.ascontiguousarray(b.T)).to(gpu).t()
    ref = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    for tile in (2, 4, 5):   # (whole tiles and rings of K steps: the persistent form runs as such)
        c = torch.empty(512, 768, dtype=torch.float32, device=gpu)
        rc = lib.mi355_gemm_tuned(ta.data_ptr(), tb.data_ptr(), c.data_ptr(), 512, 768, 1024, 1024, 1, 1, 1024, 768, 1, _lib.F32, _lib.F32,
                                  None, None, _lib.ACT_NONE, tile, 8, torch.cuda.current_stream().cuda_stream)
        assert rc == 0 and bits_equal(to_np(c), ref), tile
