"""Shared helpers for the parity tests: torch <-> float32 numpy and seeded input builders."""
from __future__ import annotations

import numpy as np
import torch

TORCH_DT = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}


def to_np(t: torch.Tensor) -> np.ndarray:
    """Any float tensor -> float32 numpy holding the same values."""
    return t.detach().float().cpu().numpy()


def from_np(x: np.ndarray, dtype: str, device) -> torch.Tensor:
    """float32 numpy holding values representable in dtype -> tensor of that dtype (exact)."""
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(TORCH_DT[dtype]).to(device)


def randn_rounded(rng: np.random.Generator, shape, dtype: str, std: float = 1.0) -> np.ndarray:
    from oracle import formats

    return formats.round_to(rng.normal(0.0, std, size=shape).astype(np.float32), dtype)


def bits_equal(a: np.ndarray, b: np.ndarray) -> bool:
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


def set_knob(monkeypatch, name: str, value) -> None:
    """Set one of the library's MI355_* environment knobs for the rest of the test.  The library reads
    the environment once per process, so it is told to read it again (conftest does the same after
    every test, when monkeypatch has restored the variables)."""
    from triton_amd import _lib

    monkeypatch.setenv(name, str(value))
    _lib.load().mi355_refresh_env()


def report_error(tag: str, got: np.ndarray, ref: np.ndarray) -> float:
    """Print (pytest -s / on failure) and return the largest |got - ref| as a fraction of max |ref|, next to the largest
    element-wise relative error over the outputs that are at least 1 % of the largest one: what the fp8 / MX tests
    actually observe under their rtol = 3e-2 bar."""
    got = np.asarray(got, dtype=np.float64); ref = np.asarray(ref, dtype=np.float64)
    top = float(np.abs(ref).max())
    d = np.abs(got - ref)
    big = np.abs(ref) >= 0.01 * top
    rel_big = float((d[big] / np.abs(ref[big])).max()) if big.any() else 0.0
    frac = float(d.max() / top) if top > 0 else 0.0
    print(f"{tag}: max |err| = {d.max():.3e} = {frac:.2e} of max |ref| ({top:.3g}); max relative error over outputs >= 1 % of it: {rel_big:.2e}")
    return frac
