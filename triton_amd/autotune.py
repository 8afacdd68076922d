"""Table-driven choice of the GEMM kernel configuration, cached per problem key.

Mirrors the control flow of the reference autotuner (python/triton/runtime/autotuner.py:146-179,
`Autotuner.run`): the key is the values of the key arguments (here M, N, K) followed by the dtype
string of every tensor argument; a key seen for the first time benchmarks every configuration with
`do_bench` (:131-133, median of the 0.5 / 0.2 / 0.8 quantiles) and stores the fastest; later calls
launch the stored configuration directly.  `TRITON_PRINT_AUTOTUNING=1` prints the same kind of line
as the reference (:168-170).  Where the reference tunes tile shape, stages and warps of a JIT
kernel (python/tutorials/03-matrix-multiplication.py:168-239), the configurations here select among
the prebuilt kernels of the library (`tile`) and the reference's GROUP_SIZE_M (`group_m`).

Extension: the table can be saved to and loaded from a JSON file, so that a serving process starts
with the choices of an earlier tuning run.
"""
from __future__ import annotations

import json
import os
import time
from dataclasses import dataclass

import torch

from . import _lib, ops, testing


@dataclass(frozen=True)
class Config:
    """One candidate (the reference's `Config`, autotuner.py:218-260, reduced to what selects a
    prebuilt kernel): `tile` as in `mi355_gemm_tuned`, `group_m` = GROUP_SIZE_M."""
    tile: int
    group_m: int = 8

    def all_kwargs(self):
        return {"tile": self.tile, "group_m": self.group_m}

    def __str__(self):
        return f"tile: {self.tile}, group_m: {self.group_m}"


def default_configs():
    """The kernels that exist for every MFMA dtype (6 falls back to 5 where its shape conditions do not hold),
    with the GROUP_SIZE_M values worth trying."""
    return [Config(1, 8), Config(2, 8), Config(3, 8), Config(4, 8), Config(5, 4), Config(5, 8), Config(5, 16),
            Config(6, 4), Config(6, 8)]


def _launch(a, b, c, config: Config, activation: int = 0):
    M, K = a.shape
    _, N = b.shape
    rc = _lib.load().mi355_gemm_tuned(
        a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K,
        a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
        ops._abi_dtype(a), ops._TORCH_TO_ABI[c.dtype], 0, 0, activation, config.tile, config.group_m, ops._stream())
    _lib.check(rc, "mi355_gemm_tuned")


class GemmAutotuner:
    """`matmul(a, b)` with the configuration looked up in (or added to) a table."""

    def __init__(self, configs=None, warmup: int = 10, rep: int = 40, bench_fn=None, cache_path: str | None = None):
        self.configs = list(configs) if configs is not None else default_configs()
        self.num_warmups, self.num_reps = warmup, rep
        # bench_fn(callable) -> milliseconds; injectable so that the table logic can be tested without a GPU
        self._bench_fn = bench_fn
        self.cache: dict[tuple, Config] = {}
        self.configs_timings: dict[Config, float] = {}
        self.best_config: Config | None = None
        self.bench_time = 0.0
        self.cache_path = cache_path
        if cache_path and os.path.exists(cache_path):
            self.load(cache_path)

    # -- the key of autotuner.py:150-158: key argument values, then one dtype string per tensor argument
    @staticmethod
    def make_key(a, b, out_dtype) -> tuple:
        M, K = a.shape
        _, N = b.shape
        return (M, N, K, str(a.dtype), str(b.dtype), str(out_dtype))

    def _bench(self, fn) -> float:
        if self._bench_fn is not None:
            return float(self._bench_fn(fn))
        q = testing.do_bench(fn, warmup=self.num_warmups, rep=self.num_reps, quantiles=(0.5, 0.2, 0.8))
        return float(q[0])

    def prune_configs(self, a, b):
        """Drop configurations that cannot differ from another one for this problem: with a single
        row or column of 256x256 tiles GROUP_SIZE_M changes nothing (the role of the reference's
        `early_config_prune`, autotuner.py:181-199)."""
        M, _ = a.shape
        _, N = b.shape
        one_dim = (M + 255) // 256 <= 1 or (N + 255) // 256 <= 1
        seen, out = set(), []
        for cfg in self.configs:
            eff = (cfg.tile, 8 if one_dim else cfg.group_m)
            if eff not in seen:
                seen.add(eff)
                out.append(cfg)
        return out

    def run(self, a, b, *, out_dtype=None, activation: str = ""):
        assert a.shape[1] == b.shape[0], "Incompatible dimensions"
        assert ops._is_contiguous(a), "Matrix A must be contiguous"
        if out_dtype is None:
            out_dtype = torch.bfloat16 if a.dtype == torch.bfloat16 else torch.float16
        act = _lib.ACT_LEAKY_RELU if activation == "leaky_relu" else _lib.ACT_NONE
        c = torch.empty((a.shape[0], b.shape[1]), device=a.device, dtype=out_dtype)
        used_cached_result = True
        if len(self.configs) > 1:
            key = self.make_key(a, b, out_dtype)
            if key not in self.cache:
                used_cached_result = False
                pruned = self.prune_configs(a, b)
                bench_start = time.time()
                timings = {cfg: self._bench(lambda cfg=cfg: _launch(a, b, c, cfg, act)) for cfg in pruned}
                self.bench_time = time.time() - bench_start
                self.cache[key] = min(timings, key=timings.get)
                self.configs_timings = timings
                if self.cache_path:
                    self.save(self.cache_path)
            config = self.cache[key]
        else:
            config = self.configs[0]
        self.best_config = config
        if os.getenv("TRITON_PRINT_AUTOTUNING", None) == "1" and not used_cached_result:
            print(f"Triton autotuning for function matmul finished after {self.bench_time:.2f}s; "
                  f"best config selected: {self.best_config};")
        _launch(a, b, c, config, act)
        return c

    __call__ = run

    # -- persistence of the table
    def save(self, path: str) -> None:
        rows = [{"key": list(k), "tile": v.tile, "group_m": v.group_m} for k, v in self.cache.items()]
        tmp = path + ".tmp"
        with open(tmp, "w") as f:
            json.dump({"version": 1, "entries": rows}, f, indent=1)
        os.replace(tmp, path)

    def load(self, path: str) -> None:
        with open(path) as f:
            doc = json.load(f)
        if doc.get("version") != 1:
            raise ValueError(f"{path}: unknown autotune table version {doc.get('version')!r}")
        for row in doc["entries"]:
            self.cache[tuple(row["key"])] = Config(int(row["tile"]), int(row["group_m"]))


_default = None


def matmul_autotuned(a, b, **kwargs):
    """`matmul(a, b)` through a process-wide `GemmAutotuner` (table file from
    `MI355_AUTOTUNE_CACHE`, if set)."""
    global _default
    if _default is None:
        _default = GemmAutotuner(cache_path=os.getenv("MI355_AUTOTUNE_CACHE") or None)
    return _default.run(a, b, **kwargs)
