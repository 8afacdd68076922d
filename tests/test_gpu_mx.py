"""GPU parity: block-scaled MXFP4 / MXFP8 matmul through the C ABI against the CPU oracle.
The reference snapshot has no MX code: the oracle here is pinned by the OCP MX v1.0 closed forms
only ("parity unpinned" by the reference); tolerance 3e-2, bit-exact where sums are exact."""
import numpy as np
import pytest
import torch

import triton_amd
from oracle import formats, mx
from util import bits_equal, report_error, to_np, set_knob

pytestmark = pytest.mark.gpu


def _operands(rng, M, N, K, fmt, lo=123, hi=132):
    if fmt == "mxfp4":
        a = rng.integers(0, 256, size=(M, K // 2)).astype(np.uint8)
        b = rng.integers(0, 256, size=(N, K // 2)).astype(np.uint8)
    else:
        fin = np.array([c for c in range(256) if c not in (0x7F, 0xFF)], dtype=np.uint8)
        a = fin[rng.integers(0, len(fin), size=(M, K))]
        b = fin[rng.integers(0, len(fin), size=(N, K))]
    sa = rng.integers(lo, hi, size=(M, K // 32)).astype(np.uint8)
    sb = rng.integers(lo, hi, size=(N, K // 32)).astype(np.uint8)
    return a, sa, b, sb


def _run(gpu, a, sa, b, sb, fmt, out_dtype):
    t = lambda x: torch.from_numpy(x).to(gpu)
    return to_np(triton_amd.mx_matmul(t(a), t(sa), t(b), t(sb), fmt, out_dtype=out_dtype))


@pytest.mark.parametrize("fmt", ["mxfp4", "mxfp8"])
@pytest.mark.parametrize("shape", [(128, 128, 256), (512, 512, 512), (300, 200, 1024), (1024, 1024, 1024),
                                   (64, 64, 96), (33, 70, 32), (256, 256, 2048), (300, 200, 1056), (128, 128, 160), (512, 256, 4064)])
def test_against_oracle(gpu, fmt, shape):
    # config 5 distribution: codes uniform, scale exponents 2^-4 .. 2^4
    M, N, K = shape
    a, sa, b, sb = _operands(np.random.default_rng(M + N + K), M, N, K, fmt)
    ref = mx.mx_matmul(a, sa, b, sb, fmt, out_dtype="bf16")
    got = _run(gpu, a, sa, b, sb, fmt, torch.bfloat16)
    scale = np.abs(ref).max()
    report_error(f"{fmt} {shape}", got, ref)
    assert np.allclose(got, ref, rtol=3e-2, atol=3e-2 * max(1.0, scale / 64))


@pytest.mark.parametrize("shape", [(256, 256, 1024), (128, 384, 4096), (130, 70, 256), (64, 64, 96), (256, 512, 1056), (130, 70, 288),
                                   (64, 64, 32), (300, 260, 2016)])     # (K / 32 odd: scale rows of odd pitch, a partial last K step)
def test_mxfp4_exact_sums_are_bitwise(gpu, shape):
    # fp4 values are multiples of 1/2 with |x| <= 6 and scales 2^-1..2^1: every product is a multiple
    # of 2^-4, every partial sum over K <= 4096 stays below 2^20 -> exact in fp32 in any order
    M, N, K = shape
    a, sa, b, sb = _operands(np.random.default_rng(7), M, N, K, "mxfp4", lo=126, hi=129)
    ref32 = mx.mx_matmul(a, sa, b, sb, "mxfp4", out_dtype="fp32")
    assert bits_equal(_run(gpu, a, sa, b, sb, "mxfp4", torch.float32), ref32)
    assert bits_equal(_run(gpu, a, sa, b, sb, "mxfp4", torch.bfloat16), formats.round_bf16(ref32))


@pytest.mark.parametrize("programs", [3, 256])
@pytest.mark.parametrize("fmt", ["mxfp4", "mxfp8"])
def test_four_wave_kernels_k_tails_are_bit_exact(gpu, monkeypatch, fmt, programs):
    # K not a multiple of 1024 in the four-wave kernels: what is left behind the last whole group of K steps follows in
    # steps whose fragments and scale bytes come straight from global memory, zeros beyond K.  Every class of tail
    # (one block, part of a step, whole steps, all but one block), one and several tiles per program (the tail runs
    # while the stages and half of the registers hold the next tile's first steps), each epilogue (fp32: general;
    # bf16, fp16: lean).  Exact data (fp4 values, or small integers as e4m3, with scales 1/2, 1, 2: every partial sum
    # is exact in fp32), so the results carry the oracle's bits.  The scale rows are slices of wider ones: the
    # 16-byte scale loads of these kernels need a pitch that is a multiple of 16.
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", programs)
    rng = np.random.default_rng(programs + len(fmt))
    M, N = 768, 512
    t = lambda x: torch.from_numpy(x).to(gpu)
    for K in (1024 + 32, 1024 + 96, 1024 + 128, 1024 + 320, 1536, 2048 + 480, 1024 + 992, 3072 + 64):
        if fmt == "mxfp4":
            a, sa, b, sb = _operands(rng, M, N, K, fmt, lo=126, hi=129)
        else:
            a = formats.encode_fp8(rng.integers(-4, 5, size=(M, K)).astype(np.float32), "e4m3")
            b = formats.encode_fp8(rng.integers(-4, 5, size=(N, K)).astype(np.float32), "e4m3")
            sa = rng.integers(126, 129, size=(M, K // 32)).astype(np.uint8)
            sb = rng.integers(126, 129, size=(N, K // 32)).astype(np.uint8)
        ref32 = mx.mx_matmul(a, sa, b, sb, fmt, out_dtype="fp32")
        pitch = -(-(K // 32) // 16) * 16
        wa = torch.full((M, pitch), 0xFF, dtype=torch.uint8, device=gpu)      # (NaN scales beyond K: never read)
        wb = torch.full((N, pitch), 0xFF, dtype=torch.uint8, device=gpu)
        wa[:, :K // 32] = t(sa)
        wb[:, :K // 32] = t(sb)
        ta, tb = t(a), t(b)
        if fmt == "mxfp8":
            ta, tb = ta.view(torch.float8_e4m3fn), tb.view(torch.float8_e4m3fn)
        for out, rnd in ((torch.float32, lambda x: x), (torch.bfloat16, formats.round_bf16), (torch.float16, lambda x: x.astype(np.float16).astype(np.float32))):
            got = to_np(triton_amd.mx_matmul(ta, wa[:, :K // 32], tb, wb[:, :K // 32], fmt, out_dtype=out))
            assert bits_equal(got, rnd(ref32)), (fmt, K, programs, out)


@pytest.mark.parametrize("programs", [3, 256])
@pytest.mark.parametrize("fmt", ["mxfp4", "mxfp8"])
def test_four_wave_kernels_on_tiles_of_192_rows_are_bit_exact(gpu, monkeypatch, fmt, programs):
    # M a multiple of 192: the four-wave block-scaled kernels also run on tiles of 192 x 256 (six A fragments per wave,
    # 48 rows of operands and scales per wave and load group; chosen by themselves where those tiles fill the CUs
    # better, forced here), one and several tiles per program, K of one to several scale-load groups.  Exact data
    # with scales 1/2, 1, 2: the oracle's bits, and those of the 256-row tiles.
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", programs)
    rng = np.random.default_rng(programs + len(fmt))
    t = lambda x: torch.from_numpy(x).to(gpu)
    for (M, N, K) in [(192, 256, 1024), (1536, 1024, 2048), (3072, 768, 1024), (576, 512, 5120), (384, 256, 3072)]:
        if fmt == "mxfp4":
            a, sa, b, sb = _operands(rng, M, N, K, fmt, lo=126, hi=129)
        else:
            a = formats.encode_fp8(rng.integers(-4, 5, size=(M, K)).astype(np.float32), "e4m3")
            b = formats.encode_fp8(rng.integers(-4, 5, size=(N, K)).astype(np.float32), "e4m3")
            sa = rng.integers(126, 129, size=(M, K // 32)).astype(np.uint8)
            sb = rng.integers(126, 129, size=(N, K // 32)).astype(np.uint8)
        ref32 = mx.mx_matmul(a, sa, b, sb, fmt, out_dtype="fp32")
        for out, rnd in ((torch.bfloat16, formats.round_bf16), (torch.float16, lambda x: x.astype(np.float16).astype(np.float32))):
            set_knob(monkeypatch, "MI355_GEMM_TILE_M", "192")
            got = _run(gpu, a, sa, b, sb, fmt, out)
            assert bits_equal(got, rnd(ref32)), (fmt, M, N, K, programs, out)
            set_knob(monkeypatch, "MI355_GEMM_TILE_M", "256")
            assert bits_equal(_run(gpu, a, sa, b, sb, fmt, out), got)
            if M % 128 == 0:   # (tiles of 128 x 256: four A fragments, 32 rows per wave and load group)
                set_knob(monkeypatch, "MI355_GEMM_TILE_M", "128")
                assert bits_equal(_run(gpu, a, sa, b, sb, fmt, out), got), "tiles of 128 rows"


@pytest.mark.parametrize("programs", [3, 256])
@pytest.mark.parametrize("fmt", ["mxfp4", "mxfp8"])
def test_two_tile_heights_in_one_launch_are_bit_exact(gpu, monkeypatch, fmt, programs):
    # the upper rows of C on 256-row tiles and the lower ones on 192-row tiles in one launch (chosen by itself for tile
    # counts that fill the last round of CUs badly, forced here): the second part starts at an offset into A, its
    # scales and C.  Exact data with scales 1/2, 1, 2: the oracle's bits, and those of one tile height.
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", programs)
    rng = np.random.default_rng(programs + len(fmt) + 7)
    for (rows256, M, N, K) in [(256, 448, 256, 1024), (256, 1216, 512, 2048), (1280, 2240, 768, 1024), (768, 960, 1024, 3072)]:
        if fmt == "mxfp4":
            a, sa, b, sb = _operands(rng, M, N, K, fmt, lo=126, hi=129)
        else:
            a = formats.encode_fp8(rng.integers(-4, 5, size=(M, K)).astype(np.float32), "e4m3")
            b = formats.encode_fp8(rng.integers(-4, 5, size=(N, K)).astype(np.float32), "e4m3")
            sa = rng.integers(126, 129, size=(M, K // 32)).astype(np.uint8)
            sb = rng.integers(126, 129, size=(N, K // 32)).astype(np.uint8)
        ref32 = mx.mx_matmul(a, sa, b, sb, fmt, out_dtype="fp32")
        for out, rnd in ((torch.bfloat16, formats.round_bf16), (torch.float16, lambda x: x.astype(np.float16).astype(np.float32))):
            set_knob(monkeypatch, "MI355_GEMM_MIXED_ROWS", rows256)
            got = _run(gpu, a, sa, b, sb, fmt, out)
            assert bits_equal(got, rnd(ref32)), (fmt, rows256, M, N, K, programs, out)
            set_knob(monkeypatch, "MI355_GEMM_MIXED_ROWS", 0)
            assert bits_equal(_run(gpu, a, sa, b, sb, fmt, out), got)


def test_scale_blocks_are_applied_per_row_and_per_32_elements(gpu):
    # all-ones data; one scale byte raised: exactly one row (or column) of C changes by 32 * (2^d - 1)
    M = N = 128; K = 512
    one4 = np.full((M, K // 2), 0x22, np.uint8)       # e2m1 code 2 = 1.0 in both nibbles
    s = np.full((M, K // 32), 127, np.uint8)
    base = _run(gpu, one4, s, one4, s, "mxfp4", torch.float32)
    assert np.all(base == K)
    for (r, kb, d) in [(5, 0, 1), (77, 9, 3), (127, 15, 2)]:
        sa = s.copy(); sa[r, kb] = 127 + d
        c = _run(gpu, one4, sa, one4, s, "mxfp4", torch.float32)
        exp = np.full((M, N), float(K), np.float32); exp[r, :] += 32 * (2.0 ** d - 1)
        assert np.array_equal(c, exp)
        c = _run(gpu, one4, s, one4, sa, "mxfp4", torch.float32)
        assert np.array_equal(c, exp.T)
    one8 = np.full((M, K), 0x38, np.uint8)            # e4m3 1.0
    for (r, kb, d) in [(3, 1, 1), (64, 7, 2), (127, 15, 4)]:
        sa = s.copy(); sa[r, kb] = 127 + d
        exp = np.full((M, N), float(K), np.float32); exp[r, :] += 32 * (2.0 ** d - 1)
        assert np.array_equal(_run(gpu, one8, sa, one8, s, "mxfp8", torch.float32), exp)
        assert np.array_equal(_run(gpu, one8, s, one8, sa, "mxfp8", torch.float32), exp.T)


def test_mfma_decodes_every_fp4_code_and_scale_exactly(gpu):
    # A[m, 0] = code m (other elements 0), B[n, 0] = 1.0: C[m, n] = e2m1(m); then every e8m0 exponent
    M = N = 128; K = 256
    a = np.zeros((M, K // 2), np.uint8); a[:16, 0] = np.arange(16)        # low nibble = element 0
    b = np.zeros((N, K // 2), np.uint8); b[:, 0] = 0x02
    s = np.full((M, K // 32), 127, np.uint8)
    c = _run(gpu, a, s, b, s, "mxfp4", torch.float32)
    assert np.array_equal(c[:16, 0], formats.e2m1_table())
    a2 = np.zeros((256, K // 2), np.uint8); a2[:, 0] = 0x02
    s2 = np.full((256, K // 32), 127, np.uint8); s2[:, 0] = np.arange(256)
    c2 = _run(gpu, a2, s2, b, s, "mxfp4", torch.float32)[:, 0]
    tab = formats.e8m0_table()
    ok = np.arange(1, 255)   # 0 is an fp32 subnormal (may flush), 255 is NaN
    assert bits_equal(c2[ok], tab[ok])
    assert np.isnan(c2[255])


@pytest.mark.parametrize("fmt", ["mxfp4", "mxfp8"])
def test_full_size_8192_sampled_rows(gpu, fmt):
    # benchmark configuration 5 at full size, checked on sampled rows against the fp64 oracle
    n = 8192
    a, sa, b, sb = _operands(np.random.default_rng(0), n, n, n, fmt)
    t = lambda x: torch.from_numpy(x).to(gpu)
    c = triton_amd.mx_matmul(t(a), t(sa), t(b), t(sb), fmt)
    assert c.dtype == torch.bfloat16 and tuple(c.shape) == (n, n)
    rows = [0, 255, 256, 4097, 8191]
    ref = mx.mx_matmul(a[rows], sa[rows], b, sb, fmt, out_dtype="bf16")
    got = to_np(c[rows])
    # (the working bar for MX is rtol = 3e-2; the absolute term, a 2000th of the largest output, only covers outputs near 0)
    report_error(f"{fmt} 8192^3, bf16 out, 5 rows", got, ref)
    assert np.allclose(got, ref, rtol=3e-2, atol=3e-2 * np.abs(ref).max() / 64)


@pytest.mark.parametrize("tile", [-1, 0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("fmt", ["mxfp4", "mxfp8"])
def test_every_kernel_variant_is_exact_on_exact_sums(gpu, monkeypatch, fmt, tile):
    # MI355_GEMM_TILE forces one kernel (-1: the one-thread-per-output kernel, an independent second implementation;
    # ping-pong, 128x128, one-barrier, pipelined 4 / 8 waves,
    # persistent) for shapes the size heuristic would give to another; K = 1536 covers three 16-byte
    # scale groups per row in the pipelined kernels (an odd number: the two-slot scale ring changes
    # parity from tile to tile in the persistent form, two programs for six and twelve tiles),
    # K = 1056 (not a multiple of 512) their fall-back.  6 = four waves of scaled 16x16x128 MFMAs (both formats): whole
    # 256x256 tiles and K a multiple of 1024 (the last two shapes: one and two groups of four K steps), else 5.
    set_knob(monkeypatch, "MI355_GEMM_TILE", str(tile))
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", "2")
    rng = np.random.default_rng(tile + 1)
    for (M, N, K) in [(512, 256, 1536), (300, 520, 1056), (768, 512, 1536), (768, 1024, 1024), (512, 256, 2048)]:
        if fmt == "mxfp4":
            a, sa, b, sb = _operands(rng, M, N, K, fmt, lo=126, hi=129)
        else:
            # e4m3 codes of small multiples of 1/2 (exact products, exact sums)
            vals = np.array([0x00, 0x30, 0x38, 0x3C, 0x40, 0xB0, 0xB8, 0xC0], dtype=np.uint8)  # 0, .5, 1, 1.5, 2, -.5, -1, -2
            a = vals[rng.integers(0, len(vals), size=(M, K))]
            b = vals[rng.integers(0, len(vals), size=(N, K))]
            sa = rng.integers(126, 129, size=(M, K // 32)).astype(np.uint8)
            sb = rng.integers(126, 129, size=(N, K // 32)).astype(np.uint8)
        ref32 = mx.mx_matmul(a, sa, b, sb, fmt, out_dtype="fp32")
        assert bits_equal(_run(gpu, a, sa, b, sb, fmt, torch.float32), ref32), (fmt, tile, M, N, K)


@pytest.mark.parametrize("fmt", ["mxfp4", "mxfp8"])
@pytest.mark.parametrize("programs", [2, 3])
def test_four_wave_kernels_deal_tiles_in_ragged_rounds(gpu, monkeypatch, fmt, programs):
    # five tiles on at most 2 / 3 programs of the scaled 16x16x128 kernels (2 + 2 + 1 tiles either way, in three or
    # two rounds); K of one and of two groups of four K steps (the scale ring's parity at the tile switch)
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", str(programs))
    rng = np.random.default_rng(60 + programs)
    for (M, N, K) in [(1280, 256, 1024), (256, 1280, 2048)]:
        if fmt == "mxfp4":
            a, sa, b, sb = _operands(rng, M, N, K, fmt, lo=126, hi=129)
        else:
            vals = np.array([0x00, 0x30, 0x38, 0x3C, 0x40, 0xB0, 0xB8, 0xC0], dtype=np.uint8)  # 0, .5, 1, 1.5, 2, -.5, -1, -2
            a = vals[rng.integers(0, len(vals), size=(M, K))]
            b = vals[rng.integers(0, len(vals), size=(N, K))]
            sa = rng.integers(126, 129, size=(M, K // 32)).astype(np.uint8)
            sb = rng.integers(126, 129, size=(N, K // 32)).astype(np.uint8)
        ref32 = mx.mx_matmul(a, sa, b, sb, fmt, out_dtype="fp32")
        assert bits_equal(_run(gpu, a, sa, b, sb, fmt, torch.float32), ref32), (fmt, programs, M, N, K)


def test_mxfp8_with_freshly_uploaded_operands_is_bit_exact_every_time(gpu, monkeypatch):
    # Regression: a tile base that the compiler had spilled was restored by a VALU instruction right in front of an
    # inline-assembly load of the four-wave MXFP8 kernel's prologue, which then - in a few per cent of launches, and
    # only with cold caches - fetched eight rows of A from a stale address.  Fresh uploads before every launch (cold
    # operands, as in the other tests' helper) and exact sums: every launch must give the bits of the oracle.
    set_knob(monkeypatch, "MI355_GEMM_TILE", "6")
    set_knob(monkeypatch, "MI355_GEMM_PROGRAMS", "5")
    rng = np.random.default_rng(65)
    M, N, K = 1280, 256, 2048
    vals = np.array([0x00, 0x30, 0x38, 0x3C, 0x40, 0xB0, 0xB8, 0xC0], dtype=np.uint8)  # 0, .5, 1, 1.5, 2, -.5, -1, -2
    cases = []
    for _ in range(3):
        a = vals[rng.integers(0, len(vals), size=(M, K))]
        b = vals[rng.integers(0, len(vals), size=(N, K))]
        sa = rng.integers(126, 129, size=(M, K // 32)).astype(np.uint8)
        sb = rng.integers(126, 129, size=(N, K // 32)).astype(np.uint8)
        cases.append((a, sa, b, sb, mx.mx_matmul(a, sa, b, sb, "mxfp8", out_dtype="fp32")))
    churn = []
    for rep in range(60):
        a, sa, b, sb, ref = cases[rep % 3]
        churn.append(torch.empty(int(rng.integers(1, 64)) * 4096, device=gpu, dtype=torch.uint8))   # moves the upload addresses around
        if len(churn) > 8:
            churn.pop(0)
        assert bits_equal(_run(gpu, a, sa, b, sb, "mxfp8", torch.float32), ref), rep


@pytest.mark.parametrize("fmt", ["mxfp4", "mxfp8"])
def test_random_shapes_through_the_default_dispatch_are_bit_exact(gpu, fmt):
    # Whatever kernel the size heuristics pick (four-wave tiles of three heights, two heights in one launch, their K
    # tails, the eight-wave kernels, partial tiles): exact data - fp4 values or small integers as e4m3, scales 1/2, 1,
    # 2 - make every partial sum exact in fp32, so the results carry the oracle's bits.  Seeded shapes around the
    # thresholds of the heuristics.
    rng = np.random.default_rng({"mxfp4": 11, "mxfp8": 12}[fmt])
    base = [64, 128, 192, 256, 384, 512, 768, 1024, 1280, 1536, 2048, 2304, 2560, 3072]
    ks = [32, 64, 256, 512, 1024, 1056, 2048, 2048 + 480, 4096]
    t = lambda x: torch.from_numpy(x).to(gpu)
    for case in range(22):
        M = int(rng.choice(base)) + int(rng.choice([0, 0, 0, 8, -8, 1]))
        N = int(rng.choice(base)) + int(rng.choice([0, 0, 0, 16, -8, 3]))
        K = int(rng.choice(ks))
        if M * N * K > 2560 * 2560 * 2048:   # (keeps the numpy oracle to about a second per case)
            K = max(32, (2560 * 2560 * 2048 // (M * N)) // 32 * 32)
        if fmt == "mxfp4":
            a, sa, b, sb = _operands(rng, M, N, K, fmt, lo=126, hi=129)
        else:
            a = formats.encode_fp8(rng.integers(-4, 5, size=(M, K)).astype(np.float32), "e4m3")
            b = formats.encode_fp8(rng.integers(-4, 5, size=(N, K)).astype(np.float32), "e4m3")
            sa = rng.integers(126, 129, size=(M, K // 32)).astype(np.uint8)
            sb = rng.integers(126, 129, size=(N, K // 32)).astype(np.uint8)
        ref32 = mx.mx_matmul(a, sa, b, sb, fmt, out_dtype="fp32")
        out = [torch.bfloat16, torch.float32, torch.float16][case % 3]
        got = to_np(triton_amd.mx_matmul(t(a), t(sa), t(b), t(sb), fmt, out_dtype=out))
        name = {torch.float32: "fp32", torch.bfloat16: "bf16", torch.float16: "fp16"}[out]
        assert bits_equal(got, formats.round_to(ref32, name)), (fmt, case, M, N, K, name)
