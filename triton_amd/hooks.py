"""Launch hooks: what profilers attach to in the reference.

The reference calls `CompiledKernel.launch_enter_hook(launch_metadata)` before and
`launch_exit_hook(launch_metadata)` after every kernel launch (python/triton/compiler/compiler.py:336-339,
third_party/amd/backend/driver.py:348-367); `launch_metadata.get()` evaluates, only when a hook asks,
the per-kernel function that the tutorials attach - `{name, flops8 | flops16, bytes}` for the matmuls
(python/tutorials/09-persistent-matmul.py:34-45).  Here the two hooks are attributes of this module's
`Launch` class and the host wrappers build the same lazily evaluated record around each C-ABI call.
With no hook set (the default) a launch pays one attribute test.
"""
from __future__ import annotations


class LaunchMetadata:
    """Lazily evaluated record: `get()` returns the dict, computing the deferred part once
    (the behaviour of the reference's LazyDict, compiler.py:318-331)."""

    def __init__(self, data: dict):
        self.data = data
        self.extras = []

    def add(self, func, args) -> None:
        self.extras.append((func, args))

    def get(self) -> dict:
        for func, args in self.extras:
            self.data = self.data | func(*args)
        self.extras.clear()
        return self.data


class Launch:
    """Holder of the two hooks (class attributes, like `CompiledKernel.launch_enter_hook`)."""
    launch_enter_hook = None
    launch_exit_hook = None


def matmul_launch_metadata(name: str, M: int, N: int, K: int, in_bytes: int) -> dict:
    """The record of python/tutorials/09-persistent-matmul.py:34-45: `flops8` for one-byte inputs,
    `flops16` otherwise (09:263-266 reads either), `bytes` = the two operands."""
    ret = {"name": f"{name} [M={M}, N={N}, K={K}]"}
    ret["flops8" if in_bytes == 1 else "flops16"] = 2.0 * M * N * K
    ret["bytes"] = in_bytes * (M * K + N * K)
    return ret


def attention_launch_metadata(name: str, Z: int, H: int, N_CTX: int, D: int, causal: bool, in_bytes: int) -> dict:
    """Forward attention in the reference's own flop count (python/tutorials/06-fused-attention.py:630-634)."""
    flops = 4.0 * Z * H * N_CTX * N_CTX * D * (0.5 if causal else 1.0)
    ret = {"name": f"{name} [Z={Z}, H={H}, N_CTX={N_CTX}, HEAD_DIM={D}, causal={bool(causal)}]"}
    ret["flops8" if in_bytes == 1 else "flops16"] = flops
    ret["bytes"] = in_bytes * 4 * Z * H * N_CTX * D
    return ret


def enter(name: str, stream: int, func, args):
    """Called by the host wrappers before a launch; returns the record for `exit` (None without hooks)."""
    if Launch.launch_enter_hook is None and Launch.launch_exit_hook is None:
        return None
    md = LaunchMetadata({"name": name, "stream": stream})
    md.add(func, args)
    if Launch.launch_enter_hook is not None:
        Launch.launch_enter_hook(md)
    return md


def exit(md) -> None:
    if md is not None and Launch.launch_exit_hook is not None:
        Launch.launch_exit_hook(md)
