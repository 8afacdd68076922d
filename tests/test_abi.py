"""CPU: the C-ABI library loads, exports exactly what include/mi355_kernels.h declares, and the
Python host surface keeps the reference's preconditions and error convention.  No kernel is
launched here."""
import ctypes
import os
import re

import pytest
import torch

import triton_amd
from triton_amd import _lib, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = open(os.path.join(ROOT, "include", "mi355_kernels.h")).read()


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for n in ("mi355_gemm", "mi355_mx_gemm", "mi355_attn_fwd", "mi355_attn_bwd_preprocess", "mi355_attn_bwd",
              "mi355_dequant", "mi355_query", "mi355_strerror"):
        assert n in names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for n in declared_functions():
        assert hasattr(lib, n), f"{n} declared in the header but not exported"


def test_binding_table_matches_header():
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_header_is_plain_c():
    # the boundary carries no torch / C++ types: compile the header as C
    import subprocess, tempfile
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.c")
        open(src, "w").write('#include "mi355_kernels.h"\nint main(void){return MI355_OK;}\n')
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", src,
                        "-o", os.path.join(d, "t.o")], check=True)


def test_strerror_and_argument_rejection_without_gpu():
    lib = _lib.load()
    assert lib.mi355_strerror(0) == b"ok"
    assert b"invalid" in lib.mi355_strerror(-1)
    # null pointers are rejected before any device work
    assert lib.mi355_gemm(None, None, None, 4, 4, 4, 4, 1, 4, 1, 4, 1, 0, 0, None, None, 0, None) == -1
    assert lib.mi355_query(12345) == -1


def test_matmul_preconditions_match_reference_messages():
    a = torch.zeros(4, 8, dtype=torch.float16)
    b = torch.zeros(6, 4, dtype=torch.float16)
    with pytest.raises(AssertionError, match="Incompatible dimensions"):   # 03:332
        triton_amd.matmul(a, b)
    with pytest.raises(AssertionError, match="Matrix A must be contiguous"):  # 03:333
        triton_amd.matmul(torch.zeros(8, 4, dtype=torch.float16).t(), torch.zeros(8, 4, dtype=torch.float16))
    with pytest.raises(AssertionError, match="Incompatible dtypes"):       # semantic.py:1355 / 09:121
        triton_amd.matmul(a, torch.zeros(8, 4, dtype=torch.bfloat16))


def test_cpu_tensor_is_a_value_error_like_the_reference_launcher():
    # third_party/amd/backend/driver.py:313-317
    a = torch.zeros(4, 8, dtype=torch.float16)
    b = torch.zeros(8, 4, dtype=torch.float16)
    with pytest.raises(ValueError, match="cannot be accessed from Triton"):
        triton_amd.matmul(a, b)


def test_attention_preconditions():
    q = torch.zeros(1, 1, 128, 48, dtype=torch.float16)
    with pytest.raises(AssertionError):      # HEAD_DIM in {16,32,64,128,256} (06:447)
        triton_amd.attention(q, q, q, True, 0.5)
    k = torch.zeros(1, 1, 128, 64, dtype=torch.float16)
    with pytest.raises(AssertionError):      # equal head dims (06:446)
        triton_amd.attention(torch.zeros(1, 1, 128, 32, dtype=torch.float16), k, k, True, 0.5)


def test_status_to_exception_mapping():
    _lib.check(0, "x")
    with pytest.raises(RuntimeError, match=r"Triton Error \[HIP\]"):   # driver.py:258-269
        _lib.check(1, "x")
    with pytest.raises(ValueError):
        _lib.check(-3, "x")


def test_dtype_names_of_reinterpreted_tensors():
    class Wrapped:   # stands in for triton.reinterpret(t, tl.float8e4nv) (jit.py:895-938)
        class dtype:
            name = "fp8e4nv"
    assert ops._abi_dtype(Wrapped()) == _lib.F8E4M3
    assert ops._abi_dtype(torch.zeros(1, dtype=torch.bfloat16)) == _lib.BF16


def test_launch_record_matches_the_tutorial_formulas():
    # python/tutorials/09-persistent-matmul.py:34-45 and 06-fused-attention.py:630-634, evaluated lazily
    from triton_amd import hooks

    calls = []

    def counted(*args):
        calls.append(args)
        return hooks.matmul_launch_metadata(*args)

    md = hooks.LaunchMetadata({"name": "k", "stream": 7})
    md.add(counted, ("k", 16, 8192, 8192, 1))
    assert calls == []                       # nothing evaluated until a hook asks
    rec = md.get()
    assert rec == {"name": "k [M=16, N=8192, K=8192]", "stream": 7, "flops8": 2.0 * 16 * 8192 * 8192,
                   "bytes": 16 * 8192 + 8192 * 8192}
    md.get()
    assert len(calls) == 1                   # and only once
    rec = hooks.attention_launch_metadata("a", 4, 32, 4096, 128, False, 2)
    assert rec["flops16"] == 2 * 2.0 * 4 * 32 * 4096 * 4096 * 128
    assert hooks.enter("x", 0, hooks.matmul_launch_metadata, ("x", 1, 1, 1, 2)) is None   # no hook set
