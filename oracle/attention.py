"""Flash-attention oracle (numpy, CPU; test infrastructure): the reference tile programs
restated, and the closed forms that pin them.

Tiled functions follow python/tutorials/06-fused-attention.py: `_attn_fwd` / `_attn_fwd_inner`
(:25-75, :98-187), `_attn_bwd_preprocess` (:190-204), `_attn_bwd_dkdv` (:208-257),
`_attn_bwd_dq` (:261-305) and the driver `_attn_bwd` (:308-435), executed one program at a time
like the interpreter's grid loop (python/triton/runtime/interpreter.py:1088-1092).  Inputs are
float32 arrays [Z, H, N, D] holding values representable in `dtype` ('fp16' | 'bf16', and for the
forward also 'e5m2' | 'e4m3': the fp8 path of 06:66-67, :609-614); rounding points use
formats.round_to(.., dtype).
"""
from __future__ import annotations

import numpy as np

from . import formats

LOG2E_FWD = 1.44269504          # the forward's literal (06:161)
RCP_LN2 = 1.4426950408889634    # the backward's literal (06:489)
LN2 = 0.6931471824645996        # 06:322


def attn_fwd_tiled(q, k, v, causal: bool, sm_scale: float, dtype: str = "fp16", BLOCK_M: int = 128, BLOCK_N: int = 64):
    """Returns (O rounded to dtype, M = m + log2(l) fp32)."""
    Z, H, N, D = q.shape
    assert N % BLOCK_M == 0 and N % BLOCK_N == 0, "the reference kernel has no bounds checks (06:98-187)"
    o = np.zeros((Z, H, N, D), dtype=np.float32)
    M = np.zeros((Z, H, N), dtype=np.float32)
    qk_scale = np.float32(np.float32(sm_scale) * np.float32(LOG2E_FWD))
    f32 = np.float32
    for hz in range(Z * H):
        z, h = hz // H, hz % H
        for start_m in range(N // BLOCK_M):
            offs_m = start_m * BLOCK_M + np.arange(BLOCK_M)
            qt = q[z, h, offs_m].astype(f32)
            m_i = np.full(BLOCK_M, -np.inf, dtype=f32)
            l_i = np.ones(BLOCK_M, dtype=f32)          # 06:157: l starts at 1, wiped by alpha = 0
            acc = np.zeros((BLOCK_M, D), dtype=f32)
            if causal:
                ranges = [(0, start_m * BLOCK_M, False), (start_m * BLOCK_M, (start_m + 1) * BLOCK_M, True)]
            else:
                ranges = [(0, N, False)]
            for lo, hi, masked in ranges:
                for start_n in range(lo, hi, BLOCK_N):
                    offs_n = start_n + np.arange(BLOCK_N)
                    kt = k[z, h, offs_n].astype(f32)
                    vt = v[z, h, offs_n].astype(f32)
                    qk = np.matmul(qt, kt.T, dtype=f32)
                    if masked:
                        mask = offs_m[:, None] >= offs_n[None, :]
                        qk = qk * qk_scale + np.where(mask, f32(0), f32(-1.0e6))
                        m_ij = np.maximum(m_i, qk.max(axis=1))
                        qk = qk - m_ij[:, None]
                    else:
                        m_ij = np.maximum(m_i, qk.max(axis=1) * qk_scale)
                        qk = qk * qk_scale - m_ij[:, None]
                    p = np.exp2(qk).astype(f32)
                    l_ij = p.sum(axis=1, dtype=f32)
                    alpha = np.exp2(m_i - m_ij).astype(f32)
                    l_i = l_i * alpha + l_ij
                    acc = acc * alpha[:, None]
                    p = formats.round_to(p, dtype)               # 06:66-69
                    acc = np.matmul(p, vt, dtype=f32) + acc
                    m_i = m_ij
            M[z, h, offs_m] = m_i + np.log2(l_i).astype(f32)
            o[z, h, offs_m] = formats.round_to(acc / l_i[:, None], dtype)
    return o, M


def attn_bwd_tiled(q, k, v, o, do, M, sm_scale: float, causal: bool = True, dtype: str = "fp16"):
    """Returns (dq, dk, dv rounded to dtype, delta fp32).

    causal=True is the reference program verbatim (its backward is causal-only: the loop bounds
    of 06:343-383 / :394-431 never look at ctx.causal).  causal=False extends both loops to the
    full range with no mask - the build's extension, pinned by attn_closed_form.
    """
    Z, H, N, D = q.shape
    f32 = np.float32
    BLOCK_M1, BLOCK_N1, BLOCK_M2, BLOCK_N2, SLICE = 32, 128, 128, 32, 2   # 06:487-488
    assert N % 128 == 0
    # host pre-scale of K, rounded to the input type (06:490-492)
    kS = formats.round_to(k.astype(f32) * f32(sm_scale * RCP_LN2), dtype)
    delta = (o.astype(f32) * do.astype(f32)).sum(axis=-1, dtype=f32)      # 06:200-204
    dq = np.zeros_like(q, dtype=f32)
    dk = np.zeros_like(q, dtype=f32)
    dv = np.zeros_like(q, dtype=f32)

    def dkdv_steps(z, h, dk_acc, dv_acc, kt, vt, offs_n, start_m, step, num_steps, mask):
        for i in range(num_steps):
            offs_m = start_m + i * step + np.arange(step)
            qT = q[z, h, offs_m].astype(f32)
            dot = do[z, h, offs_m].astype(f32)
            m = M[z, h, offs_m]
            qkT = np.matmul(kt, qT.T, dtype=f32)
            pT = np.exp2(qkT - m[None, :]).astype(f32)
            if mask:
                pT = np.where(offs_m[None, :] >= offs_n[:, None], pT, f32(0))
            dv_acc += np.matmul(formats.round_to(pT, dtype), dot, dtype=f32)
            Di = delta[z, h, offs_m]
            dpT = np.matmul(vt, dot.T, dtype=f32)
            dsT = formats.round_to(pT * (dpT - Di[None, :]), dtype)
            dk_acc += np.matmul(dsT, qT, dtype=f32)

    def dq_steps(z, h, dq_acc, qt, dot, m, Di, offs_m, start_n, step, num_steps, mask):
        for i in range(num_steps):
            offs_n = start_n + i * step + np.arange(step)
            kT = kS[z, h, offs_n].astype(f32)
            vT = v[z, h, offs_n].astype(f32)
            qk = np.matmul(qt, kT.T, dtype=f32)
            p = np.exp2(qk - m[:, None]).astype(f32)
            if mask:
                p = np.where(offs_m[:, None] >= offs_n[None, :], p, f32(0))
            dp = np.matmul(dot, vT.T, dtype=f32)
            ds = formats.round_to(p * (dp - Di[:, None]), dtype)
            dq_acc += np.matmul(ds, kT, dtype=f32)

    for hz in range(Z * H):
        z, h = hz // H, hz % H
        for pid in range(N // BLOCK_N1):
            start_n = pid * BLOCK_N1
            offs_n = start_n + np.arange(BLOCK_N1)
            kt = kS[z, h, offs_n].astype(f32)
            vt = v[z, h, offs_n].astype(f32)
            dk_acc = np.zeros((BLOCK_N1, D), dtype=f32)
            dv_acc = np.zeros((BLOCK_N1, D), dtype=f32)
            if causal:
                mb = BLOCK_M1 // SLICE
                dkdv_steps(z, h, dk_acc, dv_acc, kt, vt, offs_n, start_n, mb, BLOCK_N1 // mb, True)   # 06:346-367
                sm2 = start_n + BLOCK_N1
                dkdv_steps(z, h, dk_acc, dv_acc, kt, vt, offs_n, sm2, BLOCK_M1, (N - sm2) // BLOCK_M1, False)  # 06:369-383
            else:
                dkdv_steps(z, h, dk_acc, dv_acc, kt, vt, offs_n, 0, BLOCK_M1, N // BLOCK_M1, False)
            dv[z, h, offs_n] = formats.round_to(dv_acc, dtype)
            dk[z, h, offs_n] = formats.round_to(dk_acc * f32(sm_scale), dtype)                      # 06:385-391
            # dQ for the same 128 rows (06:394-435)
            start_m = pid * BLOCK_M2
            offs_m = start_m + np.arange(BLOCK_M2)
            qt = q[z, h, offs_m].astype(f32)
            dot = do[z, h, offs_m].astype(f32)
            m = M[z, h, offs_m]
            Di = delta[z, h, offs_m]
            dq_acc = np.zeros((BLOCK_M2, D), dtype=f32)
            if causal:
                nb = BLOCK_N2 // SLICE
                end_n = start_m + BLOCK_M2
                ns = BLOCK_M2 // nb
                dq_steps(z, h, dq_acc, qt, dot, m, Di, offs_m, end_n - ns * nb, nb, ns, True)        # 06:412-421
                end_n -= ns * nb
                ns = end_n // BLOCK_N2
                dq_steps(z, h, dq_acc, qt, dot, m, Di, offs_m, end_n - ns * BLOCK_N2, BLOCK_N2, ns, False)  # 06:423-431
            else:
                dq_steps(z, h, dq_acc, qt, dot, m, Di, offs_m, 0, BLOCK_N2, N // BLOCK_N2, False)
            dq[z, h, offs_m] = formats.round_to(dq_acc * f32(LN2), dtype)                          # 06:434
    return dq, dk, dv, delta


def attn_closed_form(q, k, v, causal: bool, sm_scale: float, do=None):
    """fp64 softmax attention and its analytic gradients (what `torch.autograd` computes for the
    reference test's materialised form, 06:532-543):
        P = softmax(Q K^T * s + mask);  O = P V;  M = logsumexp(Q K^T * s) / ln 2
        dV = P^T dO;  dP = dO V^T;  dS = P * (dP - rowsum(dP * P));  dQ = s dS K;  dK = s dS^T Q
    Returns dict with o, M and, if do is given, dq, dk, dv, delta."""
    q64, k64, v64 = (np.asarray(x, dtype=np.float64) for x in (q, k, v))
    s = np.einsum("zhmd,zhnd->zhmn", q64, k64) * sm_scale
    if causal:
        N = q.shape[2]
        s = np.where(np.tril(np.ones((N, N), dtype=bool))[None, None], s, -np.inf)
    mx = s.max(axis=-1, keepdims=True)
    e = np.exp(s - mx)
    l = e.sum(axis=-1, keepdims=True)
    p = e / l
    out = {"o": p @ v64, "M": ((mx + np.log(l)) / np.log(2.0))[..., 0], "p": p}
    if do is not None:
        do64 = np.asarray(do, dtype=np.float64)
        out["dv"] = np.einsum("zhmn,zhmd->zhnd", p, do64)
        dp = np.einsum("zhmd,zhnd->zhmn", do64, v64)
        delta = (dp * p).sum(axis=-1, keepdims=True)
        ds = p * (dp - delta)
        out["dq"] = np.einsum("zhmn,zhnd->zhmd", ds, k64) * sm_scale
        out["dk"] = np.einsum("zhmn,zhmd->zhnd", ds, q64) * sm_scale
        out["delta"] = delta[..., 0]
    return out
