"""GEMM oracle (numpy, CPU; test infrastructure): the reference tile program restated, and
the closed form that pins it.

`matmul_tiled` follows `matmul_kernel` (python/tutorials/03-matrix-multiplication.py:241-316)
as executed by the interpreter's serial grid loop (python/triton/runtime/interpreter.py:1088-1092)
with `tl.dot` = `np.matmul(a, b, dtype=float32) + acc` per K chunk (:542-549).
Arrays are float32 holding values already representable in the input type; outputs are float32
holding the rounded result (see formats.round_to).
"""
from __future__ import annotations

import numpy as np

from . import formats


def cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def grouped_pid_to_tile(pid: int, M: int, N: int, BM: int, BN: int, GROUP_M: int):
    """pid -> (pid_m, pid_n), grouped ordering (03:265-273)."""
    num_pid_m, num_pid_n = cdiv(M, BM), cdiv(N, BN)
    num_pid_in_group = GROUP_M * num_pid_n
    group_id = pid // num_pid_in_group
    first_pid_m = group_id * GROUP_M
    group_size_m = min(num_pid_m - first_pid_m, GROUP_M)
    pid_m = first_pid_m + ((pid % num_pid_in_group) % group_size_m)
    pid_n = (pid % num_pid_in_group) // group_size_m
    return pid_m, pid_n


def leaky_relu(x: np.ndarray) -> np.ndarray:
    """03:320-322 on the fp32 accumulator."""
    return np.where(x >= 0, x, np.float32(0.01) * x).astype(np.float32)


def matmul_tiled(a: np.ndarray, b: np.ndarray, BM: int = 64, BN: int = 64, BK: int = 32, GROUP_M: int = 8,
                 activation: str = "", out_dtype: str = "fp16", alpha: float = 1.0) -> np.ndarray:
    """C = A @ B tile by tile, exactly in the reference's program order.

    Row/column offsets of edge tiles wrap with % M / % N (03:282-283) and the store is masked
    (03:312-316); the K tail is zero-filled (03:297-298); one fp32 add of the chunk product per
    K step (03:300); activation on the accumulator (03:306-307); cast on store (03:308).
    `alpha` is the per-tensor scale product a_scale*b_scale of the fp8 extension (1.0 = reference).
    """
    M, K = a.shape
    K2, N = b.shape
    assert K == K2, "Incompatible dimensions"
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    c = np.zeros((M, N), dtype=np.float32)
    n_prog = cdiv(M, BM) * cdiv(N, BN)
    offs_k = np.arange(BK)
    for pid in range(n_prog):  # GridExecutor: serial loop over the 1-D grid
        pid_m, pid_n = grouped_pid_to_tile(pid, M, N, BM, BN, GROUP_M)
        offs_am = (pid_m * BM + np.arange(BM)) % M
        offs_bn = (pid_n * BN + np.arange(BN)) % N
        acc = np.zeros((BM, BN), dtype=np.float32)
        for k in range(cdiv(K, BK)):
            ks = k * BK + offs_k
            kmask = ks < K
            ksafe = np.where(kmask, ks, 0)
            at = np.where(kmask[None, :], a[offs_am[:, None], ksafe[None, :]], np.float32(0))
            bt = np.where(kmask[:, None], b[ksafe[:, None], offs_bn[None, :]], np.float32(0))
            acc = np.matmul(at, bt, dtype=np.float32) + acc
        if alpha != 1.0:
            acc = acc * np.float32(alpha)
        if activation == "leaky_relu":
            acc = leaky_relu(acc)
        out = formats.round_to(acc, out_dtype)
        offs_cm = pid_m * BM + np.arange(BM)
        offs_cn = pid_n * BN + np.arange(BN)
        mm, nn = offs_cm < M, offs_cn < N
        c[np.ix_(offs_cm[mm], offs_cn[nn])] = out[np.ix_(mm, nn)]
    return c


def matmul_closed_form(a: np.ndarray, b: np.ndarray, activation: str = "", out_dtype: str = "fp32",
                       alpha: float = 1.0) -> np.ndarray:
    """fp64 matmul of the (exactly representable) inputs, then one rounding: the golden of the
    reference's own tests (`torch.matmul(a.float(), b.float())`, hopper/test_gemm.py:138-140)."""
    acc = (np.asarray(a, dtype=np.float64) @ np.asarray(b, dtype=np.float64)) * alpha
    if activation == "leaky_relu":
        acc = np.where(acc >= 0, acc, 0.01 * acc)
    return formats.round_to(acc.astype(np.float32), out_dtype)


def dot_epilogue(a: np.ndarray, b: np.ndarray, add: np.ndarray | None = None, activation: str = "",
                 softmax: bool = False, chain_w: np.ndarray | None = None, mid_dtype: str = "fp16",
                 out_dtype: str = "fp32", alpha: float = 1.0) -> np.ndarray:
    """The epilogue chain of the reference's dot test kernel
    (python/test/unit/language/test_core.py:3128-3145) on the fp32 accumulator z = a @ b:
    `z += Z` with Z a matrix (ADD_MATRIX, :3129-3130), a per-row value broadcast along N (ADD_ROWS,
    :3131-3133) or a per-column value broadcast along M (ADD_COLS, :3134-3135) - here one `add`
    broadcastable to [M, N]; the ACTIVATION hook of the matmul tutorial
    (python/tutorials/03-matrix-multiplication.py:304-307); row softmax `exp(z - max) / sum`
    (DO_SOFTMAX, :3136-3141); `dot(z.to(w.dtype), w)` (CHAIN_DOT, :3142-3144: z is rounded to the
    operand type `mid_dtype` first).  One rounding to `out_dtype` at the store (:3145).
    Pinned by tests/test_oracle_gemm.py: zero addend = plain product, softmax rows sum to one and are
    invariant under a per-row addend, identity chain = the rounded product, and the reference's own
    z_ref formulas (:3226-3250) on integer data."""
    z = (np.asarray(a, dtype=np.float64) @ np.asarray(b, dtype=np.float64)) * alpha
    z = z.astype(np.float32)
    if add is not None:
        z = z + np.broadcast_to(np.asarray(add, dtype=np.float32), z.shape)
    if activation == "leaky_relu":
        z = leaky_relu(z)
    if softmax:
        num = np.exp(z - np.max(z, axis=1, keepdims=True))
        z = (num / np.sum(num, axis=1, keepdims=True)).astype(np.float32)
    if chain_w is not None:
        zm = formats.round_to(z, mid_dtype)
        z = (zm.astype(np.float64) @ np.asarray(chain_w, dtype=np.float64)).astype(np.float32)
    return formats.round_to(z, out_dtype)


def grouped_tile_walk(sizes, BM: int, BN: int, num_programs: int):
    """The tile schedule of `grouped_matmul_kernel` (python/tutorials/08-grouped-gemm.py:86-134):
    tiles are numbered problem after problem, row major inside a problem; program b visits
    tiles b, b + num_programs, ...  Returns, per program, the list of (problem, tile_m, tile_n)."""
    walks = []
    for b in range(num_programs):
        tile_idx, last_problem_end, visited = b, 0, []
        for g, (gm, gn, _gk) in enumerate(sizes):
            num_n_tiles = cdiv(gn, BN)
            num_tiles = cdiv(gm, BM) * num_n_tiles
            while last_problem_end <= tile_idx < last_problem_end + num_tiles:
                t = tile_idx - last_problem_end
                visited.append((g, t // num_n_tiles, t % num_n_tiles))
                tile_idx += num_programs
            last_problem_end += num_tiles
        walks.append(visited)
    return walks


def grouped_matmul(group_a, group_b, BM: int = 128, BN: int = 128, BK: int = 32, num_programs: int = 84,
                   out_dtype: str = "fp16"):
    """`group_gemm_fn` (08:143-187) executed program by program in the order of `grouped_tile_walk`:
    every tile accumulates `np.matmul(a, b, dtype=float32)` per K chunk (interpreter.py:542-549)
    and is rounded once to the output type.  Partial tiles are clipped (the reference assumes full
    tiles, 08:118 and :130)."""
    sizes = [(a.shape[0], b.shape[1], a.shape[1]) for a, b in zip(group_a, group_b)]
    outs = [np.zeros((m, n), dtype=np.float32) for (m, n, _k) in sizes]
    done = [np.zeros((cdiv(m, BM), cdiv(n, BN)), dtype=np.int32) for (m, n, _k) in sizes]
    for visited in grouped_tile_walk(sizes, BM, BN, num_programs):
        for g, tm, tn in visited:
            a = np.asarray(group_a[g], dtype=np.float32)
            b = np.asarray(group_b[g], dtype=np.float32)
            m0, n0, K = tm * BM, tn * BN, a.shape[1]
            acc = np.zeros((min(BM, a.shape[0] - m0), min(BN, b.shape[1] - n0)), dtype=np.float32)
            for k0 in range(0, K, BK):
                acc = np.matmul(a[m0:m0 + BM, k0:k0 + BK], b[k0:k0 + BK, n0:n0 + BN], dtype=np.float32) + acc
            outs[g][m0:m0 + BM, n0:n0 + BN] = formats.round_to(acc, out_dtype)
            done[g][tm, tn] += 1
    assert all((d == 1).all() for d in done), "every tile exactly once"
    return outs
