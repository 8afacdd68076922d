"""Autotune table: key, cache and persistence logic on the CPU (bench injected, launches stubbed)
and, on the GPU, tuned launches through mi355_gemm_tuned against the default path."""
import json

import numpy as np
import pytest
import torch

from triton_amd import autotune


class _FakeTensor:
    def __init__(self, shape, dtype):
        self.shape, self.dtype, self.device = shape, dtype, "cpu"

    def stride(self, i=None):
        s = (self.shape[1], 1)
        return s if i is None else s[i]


def _stub(monkeypatch, launches):
    monkeypatch.setattr(autotune, "_launch", lambda a, b, c, cfg, act=0: launches.append(cfg))
    monkeypatch.setattr(autotune.ops, "_is_contiguous", lambda t: True)
    monkeypatch.setattr(torch, "empty", lambda shape, device=None, dtype=None: _FakeTensor(shape, dtype))


def test_key_follows_the_reference_layout():
    # autotuner.py:150-158: key argument values first, then one dtype string per tensor argument
    a, b = _FakeTensor((512, 256), torch.float16), _FakeTensor((256, 1024), torch.float16)
    assert autotune.GemmAutotuner.make_key(a, b, torch.float16) == (512, 1024, 256, "torch.float16", "torch.float16", "torch.float16")


def test_first_call_benchmarks_every_config_then_the_table_answers(monkeypatch, tmp_path, capsys):
    launches = []
    _stub(monkeypatch, launches)
    cost = {1: 3.0, 2: 2.0, 3: 0.5, 4: 1.0, 5: 0.9, 6: 0.8}
    benched = []

    def bench(fn):
        fn()                       # one launch per measurement
        cfg = launches[-1]
        benched.append(cfg)
        return cost[cfg.tile] + 0.01 * cfg.group_m
    path = str(tmp_path / "table.json")
    t = autotune.GemmAutotuner(bench_fn=bench, cache_path=path)
    a, b = _FakeTensor((4096, 4096), torch.bfloat16), _FakeTensor((4096, 4096), torch.bfloat16)
    monkeypatch.setenv("TRITON_PRINT_AUTOTUNING", "1")
    t.run(a, b)
    assert [c.tile for c in benched] == [c.tile for c in t.configs] and t.best_config == autotune.Config(3, 8)
    assert launches[-1] == autotune.Config(3, 8) and len(launches) == len(t.configs) + 1
    assert "best config selected: tile: 3, group_m: 8" in capsys.readouterr().out
    n = len(launches)
    t.run(a, b)                                            # second call: no benchmark, one launch
    assert len(launches) == n + 1 and len(benched) == len(t.configs)
    assert capsys.readouterr().out == ""
    t.run(_FakeTensor((4096, 2048), torch.bfloat16), _FakeTensor((2048, 4096), torch.bfloat16))   # new key: tuned again
    assert len(benched) == 2 * len(t.configs) and len(t.cache) == 2
    # a single row of tiles: GROUP_SIZE_M cannot matter, duplicates are pruned
    assert [(c.tile, c.group_m) for c in t.prune_configs(_FakeTensor((128, 64), None), _FakeTensor((64, 4096), None))] == \
        [(1, 8), (2, 8), (3, 8), (4, 8), (5, 4), (6, 4)]
    # the table survives a restart
    doc = json.load(open(path))
    assert doc["version"] == 1 and len(doc["entries"]) == 2
    t2 = autotune.GemmAutotuner(bench_fn=lambda fn: pytest.fail("benchmarked a cached key"), cache_path=path)
    t2.run(a, b)
    assert t2.best_config == autotune.Config(3, 8)


def test_single_config_never_benchmarks(monkeypatch):
    launches = []
    _stub(monkeypatch, launches)
    t = autotune.GemmAutotuner(configs=[autotune.Config(1)], bench_fn=lambda fn: pytest.fail("benchmarked"))
    t.run(_FakeTensor((64, 64), torch.float16), _FakeTensor((64, 64), torch.float16))
    assert launches == [autotune.Config(1)]


@pytest.mark.gpu
def test_tuned_launches_match_the_default_path(gpu):
    import triton_amd
    from oracle import gemm
    from util import bits_equal, from_np, to_np
    rng = np.random.default_rng(9)
    for dtype, (M, N, K) in (("bf16", (512, 768, 256)), ("fp16", (300, 264, 520))):
        a = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        b = rng.integers(-2, 3, size=(K, N)).astype(np.float32)
        ta, tb = from_np(a, dtype, gpu), from_np(b, dtype, gpu)
        ref = gemm.matmul_closed_form(a, b)
        t = autotune.GemmAutotuner(warmup=1, rep=3)
        got = to_np(t.run(ta, tb, out_dtype=torch.float32))
        assert bits_equal(got, ref) and t.best_config in t.configs and len(t.configs_timings) >= 4
        assert all(np.isfinite(v) and v > 0 for v in t.configs_timings.values())
        assert bits_equal(to_np(t.run(ta, tb, out_dtype=torch.float32)), ref)      # from the table
        for cfg in t.configs:                                                        # every configuration is the same product
            c = torch.empty((M, N), device=gpu, dtype=torch.float32)
            autotune._launch(ta, tb, c, cfg)
            assert bits_equal(to_np(c), ref), cfg
    from triton_amd import _lib
    c = torch.empty((64, 64), device=gpu, dtype=torch.float32)
    x = torch.zeros((64, 64), device=gpu, dtype=torch.float16)
    rc = _lib.load().mi355_gemm_tuned(x.data_ptr(), x.data_ptr(), c.data_ptr(), 64, 64, 64, 64, 1, 64, 1, 64, 1,
                                      _lib.F16, _lib.F32, 0, 0, 0, 7, 8, 0)
    assert rc == _lib.EINVAL if hasattr(_lib, "EINVAL") else rc == -1
