"""ctypes binding of the C ABI in include/mi355_kernels.h (the only way into the HIP kernels).

There is deliberately no fallback: if the shared library has not been built, importing the
operators fails with an instruction to build it, and every non-zero status of a C call
becomes a Python exception.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_size_t, c_char_p, c_float, c_int, c_int64, c_void_p, POINTER
from pathlib import Path

# MI355_KERNELS_LIB: another build of the same library (a variant under test); default: the in-tree build
LIB_PATH = Path(os.environ.get("MI355_KERNELS_LIB") or Path(__file__).resolve().parent / "csrc" / "libmi355_kernels.so")

# enums of include/mi355_kernels.h
F16, BF16, F8E4M3, F8E5M2, F32 = 0, 1, 2, 3, 4
MXFP4, MXFP8 = 0, 1
ACT_NONE, ACT_LEAKY_RELU = 0, 1
DEQ_E4M3, DEQ_E5M2, DEQ_E2M1, DEQ_E8M0 = 0, 1, 2, 3
Q_ABI_VERSION, Q_CU_COUNT, Q_IS_GFX950, Q_LDS_BYTES, Q_CLOCK_KHZ, Q_STREAMK_WORKSPACE_BYTES, Q_WALL_CLOCK_KHZ = 0, 1, 2, 3, 4, 5, 6

I64x4 = c_int64 * 4

# MI355_ABI_VERSION of include/mi355_kernels.h that this binding was written for
ABI_VERSION = 5

# name -> (restype, argtypes); kept in one table so tests can check it against the header
SIGNATURES = {
    "mi355_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                           c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                           c_int, c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "mi355_gemm_tuned": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                 c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                 c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "mi355_gemm_splitk": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                  c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                  c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "mi355_gemm_streamk": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                   c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                   c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_size_t, c_void_p]),
    "mi355_gemm_streamk_static": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                          c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                          c_int, c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "mi355_gemm_epilogue": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                    c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                    c_int, c_int, c_void_p, c_void_p,
                                    c_void_p, c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "mi355_gemm_chain": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                 c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                 c_int, c_int, c_void_p, c_void_p,
                                 c_void_p, c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "mi355_grouped_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "mi355_mx_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                              c_int, c_int, c_int, c_int, c_int,
                              c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "mi355_attn_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_int, c_int, c_int, c_int,
                               POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), POINTER(c_int64),
                               c_float, c_int, c_int, c_void_p]),
    "mi355_attn_bwd_preprocess": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                          POINTER(c_int64), c_int, c_void_p]),
    "mi355_attn_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                               POINTER(c_int64), c_float, c_int, c_int, c_void_p]),
    "mi355_dequant": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "mi355_clock_probe": (c_int, [c_void_p, c_int, c_void_p]),
    "mi355_mfma_burn": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "mi355_query": (c_int, [c_int]),
    "mi355_refresh_env": (None, []),
    "mi355_strerror": (c_char_p, [c_int]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the kernel library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise ImportError(
                f"{LIB_PATH} is missing: build the HIP kernels first with "
                "`python -m triton_amd.build` (needs hipcc); there is no CPU fallback")
        lib = ctypes.CDLL(str(LIB_PATH))
        lib.mi355_query.restype, lib.mi355_query.argtypes = c_int, [c_int]
        have = lib.mi355_query(Q_ABI_VERSION)
        if have < ABI_VERSION:
            raise ImportError(f"{LIB_PATH} reports ABI version {have}, this binding needs {ABI_VERSION}: rebuild it with "
                              "`python -m triton_amd.build` (or point MI355_KERNELS_LIB at a current build)")
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


_ext = False


def ext():
    """The PyTorch-ROCm extension `_mi355_torch` (tensor objects in, torch's current stream, one C-ABI call
    per operator), or None when it has not been built or when MI355_KERNELS_LIB selects another build of the
    kernel library (the extension is linked to the in-tree one).  The operators then go through ctypes."""
    global _ext
    if _ext is False:
        _ext = None
        if not os.environ.get("MI355_KERNELS_LIB") and not os.environ.get("MI355_NO_TORCH_EXT"):
            load()  # the C library first: same build, and a clear error if it is missing
            try:
                from . import _mi355_torch  # noqa: PLC0415
                _ext = _mi355_torch
            except ImportError:
                _ext = None
    return _ext


def strerror(code: int) -> str:
    return load().mi355_strerror(code).decode()


def check(code: int, what: str) -> None:
    """Map a C status to the reference's exception convention
    (third_party/amd/backend/driver.py:258-269: HIP failures are RuntimeError)."""
    if code == 0:
        return
    if code > 0:
        raise RuntimeError(f"Triton Error [HIP]:  Code: {code}, Messsage: {strerror(code)} ({what})")
    raise ValueError(f"{what}: {strerror(code)} (code {code})")
