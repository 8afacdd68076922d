"""Writes the committed golden fixtures of tests/golden/ (run once, by hand, in the build container).

The reference cannot be imported here (its interpreter needs the compiled `triton._C.libtriton`,
which needs a network-fetched LLVM), so these vectors come from what pins the oracle without it:
  formats.json   every code of e4m3fn / e5m2 / e2m1 / e8m0 as fp32 bit patterns, produced by
                 torch's float8 views where torch has the format (e4m3fn, e5m2) and by the OCP MX
                 v1.0 definitions otherwise - NOT by oracle/formats.py, which the tests then
                 compare against this file;
  gemm_kat.npz   exactly-representable GEMM cases (inputs from {-2..2}, as in the reference's
                 python/test/unit/runtime/test_cublas.py:28-49) with integer-arithmetic results.
"""
import json
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    codes = torch.arange(256, dtype=torch.uint8)
    fmts = {
        "e4m3": codes.view(torch.float8_e4m3fn).float().numpy().view(np.uint32).tolist(),
        "e5m2": codes.view(torch.float8_e5m2).float().numpy().view(np.uint32).tolist(),
        # OCP MX v1.0 table 5 (e2m1) and section 5.4.1 (e8m0), written out by hand
        "e2m1": np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0],
                         dtype=np.float32).view(np.uint32).tolist(),
        "e8m0": [(0x00400000 if b == 0 else (b << 23)) if b != 255 else 0x7FC00000 for b in range(256)],
    }
    with open(os.path.join(HERE, "formats.json"), "w") as f:
        json.dump(fmts, f)

    rng = np.random.default_rng(1234)
    cases = {}
    for i, (M, N, K) in enumerate([(64, 64, 64), (100, 72, 40), (256, 128, 192), (33, 17, 8)]):
        a = rng.integers(-2, 3, size=(M, K)).astype(np.int64)
        b = rng.integers(-2, 3, size=(K, N)).astype(np.int64)
        cases[f"a{i}"] = a.astype(np.int8)
        cases[f"b{i}"] = b.astype(np.int8)
        cases[f"c{i}"] = (a @ b).astype(np.int32)
    np.savez_compressed(os.path.join(HERE, "gemm_kat.npz"), **cases)


if __name__ == "__main__":
    main()
