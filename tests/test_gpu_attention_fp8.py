"""GPU parity: fp8 flash-attention forward (q, k, v in e5m2 as in the reference's fp8 benchmark,
python/tutorials/06-fused-attention.py:609-614, or e4m3fn; V transposed in memory; P and O rounded
to the fp8 type, :66-67) through the C ABI against the CPU oracle.  The reference has no numeric
test of this path; the bar here: the base-2 log-sum-exp M within 1e-2, and O within one fp8 code
step of the oracle's O, or 0.01 absolutely where O crosses zero (two 2- or 3-bit roundings sit
between the fp32 sums and the output)."""
import numpy as np
import pytest
import torch

import triton_amd
from oracle import attention as A
from oracle import formats

from util import set_knob

pytestmark = pytest.mark.gpu
TDT = {"e5m2": torch.float8_e5m2, "e4m3": torch.float8_e4m3fn}


def _fp8_inputs(seed, shape, fmt, gpu):
    rng = np.random.default_rng(seed)
    codes = [formats.encode_fp8(rng.normal(0, 0.5, shape).astype(np.float32), fmt) for _ in range(3)]
    vals = [formats.fp8_table(fmt)[c].astype(np.float32) for c in codes]
    tq, tk, tv = (torch.from_numpy(c).to(gpu).view(TDT[fmt]) for c in codes)
    tv = tv.permute(0, 1, 3, 2).contiguous().permute(0, 1, 3, 2)   # 06:612-613
    return vals, (tq, tk, tv)


def _code_distance(got_codes, ref_vals, fmt):
    """|index(got) - index(ref)| on the ordered list of finite fp8 values."""
    tab = formats.fp8_table(fmt).astype(np.float64)
    finite = np.sort(np.unique(tab[np.isfinite(tab)]))
    gi = np.searchsorted(finite, tab[got_codes].astype(np.float64))
    ri = np.searchsorted(finite, ref_vals.astype(np.float64))
    return np.abs(gi - ri)


@pytest.mark.parametrize("fmt", ["e5m2", "e4m3"])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("shape", [(1, 2, 128, 64), (1, 2, 256, 128), (2, 3, 512, 128), (1, 1, 384, 64), (1, 2, 384, 128),
                                   (1, 2, 256, 16), (2, 2, 384, 32), (1, 2, 256, 256), (2, 1, 384, 256)])   # (all five head dims of 06:447)
def test_fp8_forward_against_oracle(gpu, fmt, causal, shape):
    (q, k, v), (tq, tk, tv) = _fp8_inputs(sum(shape), shape, fmt, gpu)
    sm_scale = shape[-1] ** -0.5
    o = triton_amd.attention(tq, tk, tv, causal, sm_scale)
    assert o.dtype == TDT[fmt] and o.shape == tq.shape
    ro, rM = A.attn_fwd_tiled(q, k, v, causal, sm_scale, dtype=fmt)
    codes = o.view(torch.uint8).cpu().numpy()
    got = formats.fp8_table(fmt)[codes].astype(np.float32)
    dist = _code_distance(codes, ro, fmt)
    # one code step, except around zero where neighbouring codes are 2^-16 apart and sums cancel
    near = (dist <= 1) | (np.abs(got - ro) <= 0.01)
    assert near.mean() > 0.999, f"{(~near).sum()} outputs further than one code step"
    # a P entry that rounds the other way (S differs in its last bits between the MFMA and numpy)
    # moves an output by up to one more step
    far = (dist <= 2) | (np.abs(got - ro) <= 0.02)
    assert far.all(), f"worst code distance {dist[~far].max()}"
    assert (dist == 0).mean() > 0.5   # identical codes for most outputs; the rest are rounding ties of the last cast
    cf = A.attn_closed_form(q, k, v, causal, sm_scale)
    # against the unrounded fp64 result the fp8 rounding of P dominates (the oracle itself sits
    # 0.15 |o| + 0.035 away from it on these inputs)
    assert np.all(np.abs(got - cf["o"]) <= 0.15 * np.abs(cf["o"]) + 0.05)


@pytest.mark.parametrize("causal", [True, False])
def test_fp8_forward_eight_wave_variant_gives_the_same_codes(gpu, causal, monkeypatch):
    # MI355_ATTN_FWD_VARIANT=2: 256 query rows per K/V stream (head_dim 128); N = 384 leaves half of
    # the second block empty.  Same arithmetic per row, so the output codes are identical.
    shape = (1, 2, 384, 128)
    _, (tq, tk, tv) = _fp8_inputs(5, shape, "e5m2", gpu)
    base = triton_amd.attention(tq, tk, tv, causal, 0.1).view(torch.uint8).cpu().numpy()
    set_knob(monkeypatch, "MI355_ATTN_FWD_VARIANT", "2")
    wide = triton_amd.attention(tq, tk, tv, causal, 0.1).view(torch.uint8).cpu().numpy()
    assert np.array_equal(base, wide)


@pytest.mark.parametrize("D", [16, 32, 64, 128, 256])
def test_fp8_forward_exact_case_uniform_attention(gpu, D):
    # q = 0: every score is 0, P = 1 exactly in any format, O = mean over keys of V (causal: running mean).
    # With V constant along the keys of each column the mean is that constant: exact in fp8.
    Z, H, N = 1, 2, 256
    rng = np.random.default_rng(D)
    col = formats.fp8_table("e5m2")[formats.encode_fp8(rng.normal(0, 1, (Z, H, 1, D)).astype(np.float32), "e5m2")]
    v = np.broadcast_to(col, (Z, H, N, D)).astype(np.float32)
    tq = torch.zeros(Z, H, N, D, device=gpu, dtype=torch.float8_e5m2)
    tk = torch.from_numpy(formats.encode_fp8(rng.normal(0, 1, (Z, H, N, D)).astype(np.float32), "e5m2")).to(gpu).view(torch.float8_e5m2)
    tv = torch.from_numpy(formats.encode_fp8(v, "e5m2")).to(gpu).view(torch.float8_e5m2)
    tv = tv.permute(0, 1, 3, 2).contiguous().permute(0, 1, 3, 2)
    for causal in (True, False):
        o = triton_amd.attention(tq, tk, tv, causal, 0.5)
        got = formats.fp8_table("e5m2")[o.view(torch.uint8).cpu().numpy()]
        assert np.array_equal(got, v)


def test_fp8_forward_needs_transposed_v_and_has_no_backward(gpu):
    t = torch.zeros(1, 1, 128, 64, device=gpu, dtype=torch.float8_e5m2)
    with pytest.raises(AssertionError):
        triton_amd.attention(t, t, t, False, 0.5)          # v with D contiguous
