"""Block-scaled (OCP MX v1.0) matmul oracle (numpy, CPU; test infrastructure).

PARITY UNPINNED by the reference: the snapshot has no dot_scaled / e8m0 / e2m1 code and no test
for it.  Everything here is pinned only by the OCP closed forms (formats.e2m1_table,
formats.e8m0_table), by torch's float8 views for the e4m3 elements, and by exactness KATs
(products of fp4 values and small power-of-two scales sum exactly in fp32 in any order).
"""
from __future__ import annotations

import numpy as np

from . import formats


def mx_dequant(data: np.ndarray, scales: np.ndarray, fmt: str) -> np.ndarray:
    """[R, K/2] packed e2m1 (fmt 'mxfp4') or [R, K] e4m3 codes (fmt 'mxfp8') with e8m0 scales
    [R, K/32] -> float64 [R, K]:  x[r,k] = 2^(s[r,k//32]-127) * decode(code[r,k])."""
    if fmt == "mxfp4":
        vals = formats.e2m1_table()[formats.unpack_fp4(data)]
    elif fmt == "mxfp8":
        vals = formats.fp8_table("e4m3")[data]
    else:
        raise ValueError(fmt)
    sc = formats.e8m0_table()[scales].astype(np.float64)
    assert vals.shape[1] == scales.shape[1] * 32, "one scale per 32 elements along K"
    return vals.astype(np.float64) * np.repeat(sc, 32, axis=1)


def mx_matmul(a: np.ndarray, sa: np.ndarray, b: np.ndarray, sb: np.ndarray, fmt: str,
              out_dtype: str = "bf16") -> np.ndarray:
    """C[m,n] = sum_kb 2^(sa[m,kb]-127) 2^(sb[n,kb]-127) sum_{k in kb} A^[m,k] B^[n,k], fp64
    accumulation, one rounding to out_dtype.  A is [M,K], B is [N,K] (both K-contiguous)."""
    c = mx_dequant(a, sa, fmt) @ mx_dequant(b, sb, fmt).T
    return formats.round_to(c.astype(np.float32), out_dtype)
