"""CPU: the GEMM oracle pinned by brute force, closed forms and exact known-answer cases."""
import os

import numpy as np
import pytest

from oracle import formats, gemm

KAT = np.load(os.path.join(os.path.dirname(__file__), "golden", "gemm_kat.npz"))


@pytest.mark.parametrize("M,N,BM,BN,G", [(512, 512, 64, 64, 8), (300, 200, 64, 32, 8), (1000, 130, 128, 64, 3),
                                         (64, 64, 64, 64, 8), (257, 513, 32, 32, 5)])
def test_grouped_pid_mapping_is_a_bijection_in_reference_order(M, N, BM, BN, G):
    nm, nn = gemm.cdiv(M, BM), gemm.cdiv(N, BN)
    seen = {}
    for pid in range(nm * nn):
        pm, pn = gemm.grouped_pid_to_tile(pid, M, N, BM, BN, G)
        assert 0 <= pm < nm and 0 <= pn < nn
        seen[(pm, pn)] = pid
    assert len(seen) == nm * nn
    # brute-force definition of the grouped order (03:144-150 "super-grouping"): walk groups of
    # G tile rows; inside a group go down the rows first, then one column right
    order = []
    for first in range(0, nm, G):
        rows = range(first, min(first + G, nm))
        for pn in range(nn):
            for pm in rows:
                order.append((pm, pn))
    assert [seen[t] for t in order] == list(range(nm * nn))


@pytest.mark.parametrize("i", range(4))
def test_tiled_oracle_exact_on_golden_integer_cases(i):
    a, b, c = KAT[f"a{i}"].astype(np.float32), KAT[f"b{i}"].astype(np.float32), KAT[f"c{i}"]
    for tiles in [(64, 64, 32, 8), (32, 16, 16, 2), (16, 64, 64, 1)]:
        out = gemm.matmul_tiled(a, b, *tiles, out_dtype="fp32")
        assert np.array_equal(out, c.astype(np.float32))
    assert np.array_equal(gemm.matmul_closed_form(a, b), c.astype(np.float32))


def test_single_nonzero_checks_tile_addressing_and_edge_wrap():
    M, N, K = 130, 70, 50   # edge tiles in both dims, K tail
    for (i, k, j) in [(0, 0, 0), (129, 49, 69), (64, 33, 64), (127, 48, 31)]:
        a = np.zeros((M, K), np.float32); b = np.zeros((K, N), np.float32)
        a[i, k] = 3.0; b[k, j] = -2.0
        out = gemm.matmul_tiled(a, b, 64, 64, 32, 8, out_dtype="fp16")
        exp = np.zeros((M, N), np.float32); exp[i, j] = -6.0
        assert np.array_equal(out, exp)


def test_config1_512_fp16_within_reference_tolerance():
    # benchmark configuration 1: 512^3 fp16, tiles 64x64x32, GROUP_M = 8; tolerance of 03:368 (atol 1e-2, rtol 0)
    rng = np.random.default_rng(0)
    a = formats.round_fp16(rng.standard_normal((512, 512)).astype(np.float32))
    b = formats.round_fp16(rng.standard_normal((512, 512)).astype(np.float32))
    tiled = gemm.matmul_tiled(a, b, 64, 64, 32, 8, out_dtype="fp16")
    gold = gemm.matmul_closed_form(a, b, out_dtype="fp32")
    # every output is within half an fp16 ulp (of the result) plus fp32 accumulation noise
    ulp = np.maximum(np.abs(gold), 2.0 ** -14) * 2.0 ** -11
    assert np.all(np.abs(tiled - gold) <= ulp + 1e-3)
    # the reference compares two fp16 results (03:357-371); against the fp16-rounded golden the
    # tiled result is identical except where fp32 accumulation order moved a value across a tie
    gold16 = formats.round_fp16(gold)
    assert np.mean(tiled == gold16) > 0.995
    ulp16 = np.spacing(np.abs(gold16).astype(np.float16)).astype(np.float32)
    assert np.all(np.abs(tiled - gold16) <= ulp16 + 1e-4)  # at most one fp16 ulp
    pre = gemm.matmul_tiled(a, b, 64, 64, 32, 8, out_dtype="fp32")
    # before the output rounding only fp32 accumulation noise separates it from the fp64 golden:
    # K * eps * |a| * |b| ~ 512 * 6e-8 * 1 = 3e-5 in the worst case
    assert np.max(np.abs(pre - gold)) < 1e-4


def test_leaky_relu_and_alpha_and_bf16_rounding():
    rng = np.random.default_rng(3)
    a = formats.round_bf16(rng.standard_normal((96, 80)).astype(np.float32))
    b = formats.round_bf16(rng.standard_normal((80, 72)).astype(np.float32))
    out = gemm.matmul_tiled(a, b, 32, 32, 32, 4, activation="leaky_relu", out_dtype="bf16", alpha=0.5)
    gold = gemm.matmul_closed_form(a, b, activation="leaky_relu", out_dtype="bf16", alpha=0.5)
    # identical up to one bf16 ulp where the fp32 accumulation order moved a value across a tie
    assert np.max(np.abs(out - gold) / np.maximum(np.abs(gold), 1e-3)) <= 2.0 ** -7
    x = np.array([[-4.0, 2.0]], np.float32)
    assert np.array_equal(gemm.leaky_relu(x), np.array([[-0.04, 2.0]], np.float32))


def test_linearity_and_identity():
    rng = np.random.default_rng(4)
    a = rng.integers(-3, 4, size=(70, 64)).astype(np.float32)
    eye = np.eye(64, dtype=np.float32)
    assert np.array_equal(gemm.matmul_tiled(a, eye, 32, 32, 16, 8, out_dtype="fp32"), a)
    perm = eye[:, rng.permutation(64)]
    assert np.array_equal(gemm.matmul_tiled(a, perm, 32, 32, 16, 8, out_dtype="fp32"), a @ perm)


def test_dot_epilogue_pins():
    # the epilogue chain of the reference's dot test (test_core.py:3128-3145) against what the
    # mathematics fixes and against the reference's own z_ref formulas (:3226-3250) on integer data
    rng = np.random.default_rng(17)
    M, N, K = 48, 40, 24
    a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    b = rng.integers(-3, 4, size=(K, N)).astype(np.float32)
    z0 = rng.integers(-5, 6, size=(M, N)).astype(np.float32)
    plain = gemm.matmul_closed_form(a, b)
    assert np.array_equal(gemm.dot_epilogue(a, b, add=np.zeros((M, N), np.float32)), plain)
    # z_ref += z ; z_ref += z[:, 0][:, None] ; z_ref += z[0, :][None, :]   (exact in integers)
    assert np.array_equal(gemm.dot_epilogue(a, b, add=z0), a @ b + z0)
    assert np.array_equal(gemm.dot_epilogue(a, b, add=z0[:, :1]), a @ b + z0[:, 0][:, None])
    assert np.array_equal(gemm.dot_epilogue(a, b, add=z0[:1, :]), a @ b + z0[0, :][None, :])
    # a transposed broadcast (rows taken for columns) must fail the comparison above: M != N
    # softmax: rows sum to one, invariant under a per-row addend, equal to the reference formula
    s = gemm.dot_epilogue(0.1 * a, 0.1 * b, softmax=True)
    assert np.allclose(s.sum(axis=1), 1.0, atol=1e-6) and np.all(s > 0)
    assert np.allclose(gemm.dot_epilogue(0.1 * a, 0.1 * b, add=z0[:, :1], softmax=True), s, atol=1e-6)
    zr = (0.1 * a) @ (0.1 * b)
    num = np.exp(zr - np.max(zr, axis=-1, keepdims=True))
    assert np.allclose(s, num / np.sum(num, axis=-1, keepdims=True), atol=1e-6)
    assert not np.allclose(gemm.dot_epilogue(0.1 * a, 0.1 * b, add=z0[:1, :], softmax=True), s, atol=1e-3)
    # chain-dot: identity W returns the rounded product; integer W is exact
    eye = np.eye(N, dtype=np.float32)
    assert np.array_equal(gemm.dot_epilogue(a, b, chain_w=eye), formats.round_to(plain, "fp16"))
    w = rng.integers(-2, 3, size=(N, N)).astype(np.float32)
    assert np.array_equal(gemm.dot_epilogue(a, b, chain_w=w), (a @ b) @ w)
    # the intermediate rounding is visible: bf16 keeps 8 bits of 257
    a1 = np.full((1, 1), 257.0, np.float32)
    one = np.ones((1, 1), np.float32)
    assert gemm.dot_epilogue(a1, one, chain_w=one, mid_dtype="bf16")[0, 0] == 256.0
    assert gemm.dot_epilogue(a1, one, chain_w=one, mid_dtype="fp16")[0, 0] == 257.0
