"""Benchmark of the hot path on one MI355X.

`python bench.py --gpus 1 --steps K --warmup W` times K back-to-back launches of the headline
workload (bf16 GEMM 8192^3, benchmark configuration 2) with inputs resident in HBM, and prints ONE JSON
line: TFLOP/s (work = 2*M*N*K as in python/tutorials/03-matrix-multiplication.py:437), the MFMA
roofline fraction of the GEMM kernel from per-launch device events, and the CPU oracle timed on
the host cores.  The other workloads of the path (fp8 / MX GEMM, attention forward / backward)
are timed briefly and reported under "extra".
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# dense MFMA peaks of MI355X in TFLOP/s (published, without sparsity) and HBM3E bandwidth in GB/s
PEAK = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "mxfp8": 5000.0, "mxfp4": 10100.0, "fp32": 157.3}
HBM_GBPS = 8000.0

# HBM-side bytes per launch of the 8192^3 bf16 GEMM kernel.  NOT read in this run (hardware counters need
# rocprofv3 around the process): taken from the two rocprofv3 --pmc runs of this same command that
# profiles/gemm_bf16_8192.md records - FETCH_SIZE and WRITE_SIZE in KiB per dispatch, each scaled by what
# the same counter reads for a plain device copy of known size (--copy-calibration).
MEASURED_TRAFFIC_KIB = {"FETCH_SIZE": 844913, "FETCH_scale": 2.000, "WRITE_SIZE": 136400, "WRITE_scale": 1.000}   # medians over > 1100 dispatches
MEASURED_TRAFFIC_BYTES = int((MEASURED_TRAFFIC_KIB["FETCH_SIZE"] * MEASURED_TRAFFIC_KIB["FETCH_scale"]
                              + MEASURED_TRAFFIC_KIB["WRITE_SIZE"] * MEASURED_TRAFFIC_KIB["WRITE_scale"]) * 1024)
TRAFFIC_SOURCE = "profiles/gemm_bf16_8192.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, separate runs of this command; not measured in this run)"


def time_launches(fn, steps, warmup):
    """W untimed warm-up launches, then exactly K launches timed two ways: wall clock between two
    device synchronisations, and K+1 device events on the launch stream (per-launch durations)."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(steps):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    per = [ev[i].elapsed_time(ev[i + 1]) for i in range(steps)]
    return wall_ms, sum(per) / len(per), per


def settle(fn, seconds=0.06, limit=4000):
    """Untimed launches for `seconds` of wall time (at most `limit` of them): after a change of kernel, and more so
    after an idle phase, the board takes tens of milliseconds to settle its clocks - the first 10 launches of the
    8192^3 GEMM read 3 % below what follows, 40 launches of the 0.25 ms grouped GEMM 14 % (975 against 1110-1130
    TFLOP/s), and the 15-30 us skinny kernels never got there within their warm-up launches."""
    import torch

    t0 = time.perf_counter()
    done = 0
    while done < limit and time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        done += 20
        torch.cuda.synchronize()
    return done


def quick(fn, iters=60, warmup=20):
    settle(fn)
    _, ev_ms, _ = time_launches(fn, iters, warmup)
    return ev_ms


def observed_board_state(fn, seconds=1.0):
    """Shader clock and board power while `fn` runs back to back (an untimed leg of its own), from the driver's
    own files: the current-clock line of /sys/class/drm/card*/device/pp_dpm_sclk (what rocm-smi --showclocks
    prints) and hwmon's power1_average / power1_input with power1_cap (microwatts; what rocm-smi --showpower /
    --showmaxpower print), sampled every 10 ms by a host thread over `seconds` of sustained launches; medians of
    the samples taken after the first quarter.  Fields that cannot be read are None.  (The board holds its power
    limit by lowering the clock of MFMA-heavy kernels, so the nominal clock says little and the watts next to
    the cap say why.  The library's own mi355_clock_probe reads the counters on the device, but a probe wave next
    to a kernel that fills every SIMD costs that kernel a round of tiles, and the clock is back up within
    microseconds of a kernel's end - so it suits kernels that leave a wave slot free, not these.)"""
    import glob
    import re
    import threading

    import torch

    clk_paths = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
    hw = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*"))
    pw_paths = [q for d in hw for q in (os.path.join(d, "power1_average"), os.path.join(d, "power1_input")) if os.path.exists(q)]
    cap = None
    for d in hw:
        try:
            cap = max(cap or 0.0, int(open(os.path.join(d, "power1_cap")).read()) / 1e6)
        except (OSError, ValueError):
            pass
    clk, watts, stop = [], [], [False]

    def read_max(paths, parse):
        best = None
        for path in paths:   # (one GPU per box; with several cards, the busiest one is the one under test)
            try:
                v = parse(open(path).read())
            except (OSError, ValueError):
                v = None
            if v is not None:
                best = max(best or 0, v)
        return best

    def sclk(text):
        m = re.search(r"(\d+)\s*Mhz\s*\*", text, re.I)
        return int(m.group(1)) if m else None

    def poll():
        while not stop[0]:
            c = read_max(clk_paths, sclk)
            w = read_max(pw_paths, lambda t: int(t) / 1e6)
            if c is not None:
                clk.append(c)
            if w is not None:
                watts.append(w)
            time.sleep(0.01)

    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    th = threading.Thread(target=poll)
    th.start()
    t0 = time.perf_counter()
    done = torch.cuda.Event()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            fn()
        done.record()
        done.synchronize()
    stop[0] = True
    th.join()
    torch.cuda.synchronize()

    def median_tail(xs):
        tail = sorted(xs[len(xs) // 4:])
        return round(float(tail[len(tail) // 2]), 1) if tail else None

    return {"sclk_mhz": median_tail(clk), "power_w": median_tail(watts), "power_cap_w": cap}


def _median_of_3(fn):
    """1 warm + median of 3 passes, seconds."""
    fn()
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[1]


def cpu_baselines_other(threads):
    """The other CPU legs: config 1 in full under the interpreter's execution model, the attention
    oracle on a (Z, H) = (1, 1) slice of config 3 (flagged: a slice, not the whole job), and plain
    multithreaded fp32 torch.matmul on the host as the best-CPU line."""
    import numpy as np
    import torch

    from oracle import attention as OA
    from oracle import formats, gemm

    out = {}
    rng = np.random.default_rng(0)
    a = formats.round_fp16(rng.standard_normal((512, 512)).astype(np.float32))
    b = formats.round_fp16(rng.standard_normal((512, 512)).astype(np.float32))
    dt = _median_of_3(lambda: gemm.matmul_tiled(a, b, 64, 64, 32, 8, out_dtype="fp16"))
    out["config1_fp16_512_tiles_64x64x32"] = {
        "value": round(2.0 * 512 ** 3 / dt / 1e12, 6), "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": f"oracle.gemm.matmul_tiled 512^3 fp16 in full (64 programs x 16 K steps, serial grid loop), 1 warm + median of 3, {dt * 1e3:.1f} ms"}
    Z, H, N, D = 1, 1, 4096, 128
    q, k, v = (formats.round_bf16(rng.normal(0, 0.5, (Z, H, N, D)).astype(np.float32)) for _ in range(3))
    for causal in (True, False):
        dt = _median_of_3(lambda: OA.attn_fwd_tiled(q, k, v, causal, D ** -0.5, "bf16"))
        fl = 4.0 * Z * H * N * N * D * (0.5 if causal else 1.0)
        out[f"attn_fwd_{'causal' if causal else 'noncausal'}"] = {
            "value": round(fl / dt / 1e12, 5), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"oracle.attention.attn_fwd_tiled bf16 on the (Z, H) = (1, 1) slice of config 3 (N=4096, D=128; 1/128 of the job, flagged: slice), "
                      f"1 warm + median of 3, {dt:.2f} s"}
    n = 4096
    ta, tb = torch.randn(n, n), torch.randn(n, n)
    dt = _median_of_3(lambda: torch.matmul(ta, tb))
    out["torch_matmul_fp32_best_cpu"] = {
        "value": round(2.0 * n ** 3 / dt / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "library",
        "sample": f"torch.matmul fp32 {n}^3 on the host (not the reference's path: the best-CPU line), 1 warm + median of 3, {dt:.2f} s"}
    return out


def cpu_baseline_gemm(budget_s=20.0):
    """The CPU oracle (a port of the reference's interpreter execution model: serial grid loop,
    one fp32 np.matmul per K chunk, python/triton/runtime/interpreter.py:1088-1092, :542-549) on a
    bounded sample of the GEMM workload: same tile program, size reduced until it fits the budget."""
    import numpy as np

    from oracle import formats, gemm

    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = os.cpu_count() or 1
    rng = np.random.default_rng(0)
    # size: the largest power of two whose four passes (1 warm + 3 timed) fit the budget, found by doubling
    n = 1024
    while True:
        a = formats.round_bf16(rng.standard_normal((n, n)).astype(np.float32))
        b = formats.round_bf16(rng.standard_normal((n, n)).astype(np.float32))
        t0 = time.perf_counter()
        gemm.matmul_tiled(a, b, 128, 256, 64, 8, out_dtype="bf16")
        dt = time.perf_counter() - t0
        if dt * 8 * 4 > budget_s or n >= 8192:
            break
        n *= 2
    dt = _median_of_3(lambda: gemm.matmul_tiled(a, b, 128, 256, 64, 8, out_dtype="bf16"))
    base = {
        "value": round(2.0 * n ** 3 / dt / 1e12, 5), "unit": "TFLOP/s", "cores": int(threads), "kind": "port",
        "sample": f"oracle.gemm.matmul_tiled {n}^3 bf16 values (tiles 128x256x64, GROUP_M 8, fp32 accumulate, bf16 out): the {n}^3 "
                  f"sub-problem of the 8192^3 workload (1/{(8192 // n) ** 3} of its flop; throughput, not extrapolated time), "
                  f"1 warm + median of 3, {dt:.2f} s per pass; BLAS threads {threads}, host has {os.cpu_count()} logical cpus",
    }
    try:
        base["other_legs"] = cpu_baselines_other(int(threads))
    except Exception as e:   # a baseline leg must never take the GPU numbers down with it
        base["other_legs"] = {"error": repr(e)}
    return base


def secondary_workloads(lib, dev, n):
    """name -> builder of the other workloads of the path.  A builder allocates its inputs (synthetic, on the
    distributions the configurations state) and returns (launch function, algorithmic flop or bytes per
    launch, "flops" | "bytes", {"peak": ..., "data": ..., "clock": bool}, launches to time)."""
    import torch

    import triton_amd
    from triton_amd import _lib

    stream = torch.cuda.current_stream().cuda_stream
    flops = 2.0 * n ** 3
    W = {}

    # config 4: N(0, 1) scaled to a per-tensor amax of 448, clamped, cast to e4m3fn; the fp32 scales that undo
    # it go to the epilogue; K-major B, bf16 out
    def quantize_e4m3(x):
        scale = (x.abs().amax() / 448.0).float().reshape(1)
        return (x / scale).clamp(-448.0, 448.0).to(torch.float8_e4m3fn), scale

    def fp8_gemm():
        a8, sa8 = quantize_e4m3(torch.randn(n, n, device=dev))
        b8, sb8 = quantize_e4m3(torch.randn(n, n, device=dev))
        fn = lambda: triton_amd.matmul(a8, b8.t(), out_dtype=torch.bfloat16, a_scale=sa8, b_scale=sb8)
        return fn, flops, "flops", {"peak": "fp8", "clock": True, "data": "N(0,1) scaled to amax 448, e4m3fn, per-tensor fp32 scales"}, 60
    W["fp8_e4m3_gemm_8192"] = fp8_gemm

    # fp32 operands on the fp32 MFMAs (the `ieee` precision of `tl.dot`): N(0, 1), K-major B as the kernel takes it,
    # fp32 out; 7 ms per launch, so a handful of launches
    def fp32_gemm():
        a32 = torch.randn(n, n, device=dev)
        b32 = torch.randn(n, n, device=dev)      # [N, K]: b32.t() is the K-major [K, N] operand
        c32 = torch.empty(n, n, device=dev)

        def fn():
            rc = lib.mi355_gemm(a32.data_ptr(), b32.data_ptr(), c32.data_ptr(), n, n, n, n, 1, 1, n, n, 1,
                                _lib.F32, _lib.F32, None, None, 0, stream)
            assert rc == 0, rc

        return fn, flops, "flops", {"peak": "fp32", "clock": True, "data": "N(0,1) fp32, K-major B, fp32 out"}, 8
    W["fp32_gemm_8192"] = fp32_gemm

    def fp8_decode():
        b8, _ = quantize_e4m3(torch.randn(n, n, device=dev))
        a16, _ = quantize_e4m3(torch.randn(16, n, device=dev))
        c16 = torch.empty(16, n, device=dev, dtype=torch.bfloat16)

        def fn():  # straight through the C ABI: at ~20 us per launch the Python wrapper would dominate
            rc = lib.mi355_gemm(a16.data_ptr(), b8.data_ptr(), c16.data_ptr(), 16, n, n, n, 1, 1, n, n, 1,
                                _lib.F8E4M3, _lib.BF16, None, None, 0, stream)
            assert rc == 0, rc

        return fn, n * n + 16 * n + 2 * 16 * n, "bytes", {}, 50
    W["fp8_decode_m16"] = fp8_decode

    # 16-bit skinny shapes of the reference's regression table (test_performance.py:36-44): fp16, row-major B
    def skinny(sm, sn, sk):
        def build():
            xa = torch.randn(sm, sk, device=dev, dtype=torch.float16)
            xb = torch.randn(sk, sn, device=dev, dtype=torch.float16)
            xc = torch.empty(sm, sn, device=dev, dtype=torch.float16)

            def fn():
                rc = lib.mi355_gemm(xa.data_ptr(), xb.data_ptr(), xc.data_ptr(), sm, sn, sk, sk, 1, sn, 1, sn, 1,
                                    _lib.F16, _lib.F16, None, None, 0, stream)
                assert rc == 0, rc

            return fn, 2 * (sm * sk + sk * sn + sm * sn), "bytes", {}, 50
        return build
    for (sm, sn, sk) in ((16, n, n), (64, n, n), (n, 64, n)):
        W[f"fp16_skinny_{sm}x{sn}x{sk}"] = skinny(sm, sn, sk)

    # the decode shape with the weight as a linear layer stores it: B[N, K], K contiguous (x @ W^T)
    def decode_kmajor():
        xa = torch.randn(16, n, device=dev, dtype=torch.float16)
        xw = torch.randn(n, n, device=dev, dtype=torch.float16)   # [N, K]
        xc = torch.empty(16, n, device=dev, dtype=torch.float16)

        def fn():
            rc = lib.mi355_gemm(xa.data_ptr(), xw.data_ptr(), xc.data_ptr(), 16, n, n, n, 1, 1, n, n, 1,
                                _lib.F16, _lib.F16, None, None, 0, stream)
            assert rc == 0, rc

        return fn, 2 * (16 * n + n * n + 16 * n), "bytes", {}, 50
    W["fp16_decode_m16_kmajor_weight"] = decode_kmajor

    # grouped GEMM (tutorial 08): 16 fp16 problems of 2048^3 in one launch; launch only, device tables prepared
    # once (like `triton_perf_fn`, 08:217-228)
    def grouped():
        ga = [torch.randn(2048, 2048, device=dev, dtype=torch.float16) for _ in range(16)]
        gb = [torch.randn(2048, 2048, device=dev, dtype=torch.float16) for _ in range(16)]
        gc = [torch.empty(2048, 2048, device=dev, dtype=torch.float16) for _ in range(16)]
        i64 = lambda xs: torch.tensor([x.data_ptr() for x in xs], device=dev, dtype=torch.int64)
        d_a, d_b, d_c = i64(ga), i64(gb), i64(gc)
        d_sz = torch.tensor([2048] * 48, device=dev, dtype=torch.int32)
        d_ld = torch.tensor([2048] * 48, device=dev, dtype=torch.int32)

        def fn(keep=(ga, gb, gc)):
            rc = lib.mi355_grouped_gemm(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr(), d_sz.data_ptr(), d_ld.data_ptr(),
                                        16, _lib.F16, 0, stream)
            assert rc == 0, rc

        return fn, 16 * 2.0 * 2048 ** 3, "flops", {"peak": "fp16"}, 60
    W["grouped_gemm_16x2048"] = grouped

    # config 5: fp4 codes uniform over all 16 values (every byte value), e4m3 codes uniform over the 254 finite
    # ones (0x7F / 0xFF are NaN), e8m0 scales uniform over 2^-4 .. 2^4
    def mx(fmt):
        def build():
            kb = n // 2 if fmt == "mxfp4" else n

            def codes():
                if fmt == "mxfp4":
                    return torch.randint(0, 256, (n, kb), device=dev, dtype=torch.uint8)
                r = torch.randint(0, 254, (n, kb), device=dev, dtype=torch.uint8)
                return r + (r >= 127).to(torch.uint8)      # 0..126 -> 0x00..0x7E, 127..253 -> 0x80..0xFE

            pa, pb = codes(), codes()
            sa = torch.randint(123, 132, (n, n // 32), device=dev, dtype=torch.uint8)
            sb = torch.randint(123, 132, (n, n // 32), device=dev, dtype=torch.uint8)
            fn = lambda: triton_amd.mx_matmul(pa, sa, pb, sb, fmt)
            return fn, flops, "flops", {"peak": fmt, "clock": True,
                                        "data": "codes uniform over all finite values, e8m0 scales uniform over 2^-4 .. 2^4"}, 60
        return build
    W["mxfp4_gemm_8192"] = mx("mxfp4")
    W["mxfp8_gemm_8192"] = mx("mxfp8")

    # flash attention (config 3), flops by the reference formula (06:630-636)
    Z, H, N, D = 4, 32, 4096, 128
    sm_scale = D ** -0.5

    def qkv():
        return tuple(torch.empty(Z, H, N, D, device=dev, dtype=torch.bfloat16).normal_(0, 0.5) for _ in range(3))

    def attn_fwd(causal):
        def build():
            q, k, v = qkv()
            fn = lambda: triton_amd.attention(q, k, v, causal, sm_scale)
            return fn, 4.0 * Z * H * N * N * D * (0.5 if causal else 1.0), "flops", {"peak": "bf16", "clock": True}, 60
        return build

    def attn_bwd(causal):
        def build():
            q, k, v = (t.requires_grad_() for t in qkv())
            o = triton_amd.attention(q, k, v, causal, sm_scale)
            do = torch.randn_like(o)
            # gradients returned, not accumulated into .grad (that would add three elementwise kernels)
            fn = lambda: torch.autograd.grad(o, (q, k, v), do, retain_graph=True)
            return fn, 2.5 * 4.0 * Z * H * N * N * D * (0.5 if causal else 1.0), "flops", {"peak": "bf16", "clock": True}, 8
        return build

    # fp8 forward (06:609-614): e5m2 inputs, V transposed in memory
    def attn_fwd8(causal):
        def build():
            q, k, v = qkv()
            q8, k8 = q.to(torch.float8_e5m2), k.to(torch.float8_e5m2)
            v8 = v.permute(0, 1, 3, 2).contiguous().permute(0, 1, 3, 2).to(torch.float8_e5m2)
            fn = lambda: triton_amd.attention(q8, k8, v8, causal, sm_scale)
            return fn, 4.0 * Z * H * N * N * D * (0.5 if causal else 1.0), "flops", {"peak": "fp8"}, 60
        return build

    for causal in (True, False):
        tag = "causal" if causal else "noncausal"
        W[f"attn_fwd_{tag}"] = attn_fwd(causal)
        W[f"attn_bwd_{tag}"] = attn_bwd(causal)
    for causal in (True, False):
        W[f"attn_fwd_fp8_{'causal' if causal else 'noncausal'}"] = attn_fwd8(causal)
    return W


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    # (100 launches = 75 ms: the clocks have settled by then; with 10 the timed region starts 3 % low)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="wall time of untimed launches of the headline GEMM in front of the warm-up (the board's clocks "
                         "take tens of milliseconds to settle after an idle phase); reported as settle_launches")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--size", type=int, default=8192)
    ap.add_argument("--only", default=None,
                    help="run just this secondary workload (a key of the 'extra' object) for --steps launches and print its "
                         "record: the command line to put under rocprofv3 for that workload's kernels")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch plain device copies of the A matrix (a kernel of known traffic, for scaling PMC byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the path has no collectives); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    import triton_amd
    from triton_amd import _lib

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    lib = _lib.load()
    dev = torch.device("cuda", 0)
    torch.manual_seed(0)
    n = args.size
    if args.only:
        table = secondary_workloads(lib, dev, n)
        if args.only not in table:
            print("bench.py: --only takes one of " + ", ".join(table), file=sys.stderr)
            sys.exit(2)
        fn, work, kind, info, _ = table[args.only]()
        settle(fn)
        wall_ms, ev_ms, _ = time_launches(fn, args.steps, args.warmup)
        rec = {"workload": args.only, "steps": args.steps, "ms_per_launch": round(ev_ms, 5),
               ("tflops" if kind == "flops" else "gbps"): round(work / ev_ms / (1e9 if kind == "flops" else 1e6), 1)}
        if info.get("clock"):
            rec.update(observed_board_state(fn, 0.5))
        print(json.dumps(rec))
        return
    a = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
    b = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
    c = torch.empty(n, n, device=dev, dtype=torch.bfloat16)
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        rc = lib.mi355_gemm(a.data_ptr(), b.data_ptr(), c.data_ptr(), n, n, n, n, 1, n, 1, n, 1,
                            _lib.BF16, _lib.BF16, None, None, 0, stream)
        assert rc == 0, rc

    if args.copy_calibration:
        for _ in range(5):
            c.copy_(a)   # reads n*n*2 bytes, writes n*n*2 bytes
        torch.cuda.synchronize()
    # untimed launches until the clocks have settled (as for every secondary workload), then W warm-up launches,
    # then exactly K timed ones
    settle_launches = settle(step, args.settle_ms * 1e-3)
    wall_ms, ev_ms, per = time_launches(step, args.steps, args.warmup)
    flops = 2.0 * n ** 3
    tflops = flops / (wall_ms * 1e-3) / 1e12
    achieved = flops / (ev_ms * 1e-3) / 1e12
    out = {
        "metric": "TFLOP/s & % MFMA peak: bf16/fp8 GEMM 8192^3; flash-attn fwd D=128 N=4096",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_launches": settle_launches,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"bf16 GEMM M=N=K={n}, A row-major MxK, B row-major KxN, fp32 accumulate, bf16 out (BASELINE config 2)"},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK["bf16"], "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK["bf16"], 4), "traffic": MEASURED_TRAFFIC_BYTES,
                     "kernel": "gemm_wave128_kernel<bf16, row-major B> (256x256 tiles, four waves of 128x128 from 16x16x32 MFMAs, two 64 KiB LDS stages, one program per CU)", "launch_ms_avg": round(ev_ms, 5),
                     "launch_ms_min": round(min(per), 5), "algorithmic_flops": flops,
                     "algorithmic_bytes": 3 * 2 * n * n},
        "device": {"name": torch.cuda.get_device_name(0), "cus": lib.mi355_query(_lib.Q_CU_COUNT),
                   "nominal_clock_khz": lib.mi355_query(_lib.Q_CLOCK_KHZ),
                   "during_headline_gemm": observed_board_state(step)},
    }
    out["roofline"]["traffic_source"] = TRAFFIC_SOURCE

    if not args.no_extra:
        from triton_amd import testing

        extra = {}
        # the reference's own timing protocol (cache flushed before every call, per-call events)
        med, p20, p80 = testing.do_bench(step, warmup=25, rep=100, quantiles=[0.5, 0.2, 0.8])
        extra["bf16_gemm_do_bench"] = {"ms_median": round(med, 4), "ms_p20": round(p20, 4), "ms_p80": round(p80, 4),
                                       "tflops_median": round(testing.matmul_tflops(n, n, n, med), 1)}
        del a, b, c
        # config 2's sweep: square sizes 1024 .. 8192 in steps of 1024, bf16, row-major B, the reference's protocol
        # (flushed do_bench medians, 03:424-438) through the same C-ABI call as the headline
        sweep = {}
        for m in range(1024, 8192 + 1, 1024):
            sa_, sb_ = (torch.randn(m, m, device=dev, dtype=torch.bfloat16) for _ in range(2))
            sc_ = torch.empty(m, m, device=dev, dtype=torch.bfloat16)

            def sweep_step(m=m, sa_=sa_, sb_=sb_, sc_=sc_):
                rc = lib.mi355_gemm(sa_.data_ptr(), sb_.data_ptr(), sc_.data_ptr(), m, m, m, m, 1, m, 1, m, 1,
                                    _lib.BF16, _lib.BF16, None, None, 0, stream)
                assert rc == 0, rc

            settle(sweep_step, 0.03)
            med = testing.do_bench(sweep_step, warmup=10, rep=40, quantiles=[0.5])
            sweep[str(m)] = {"ms_median": round(med, 4), "tflops": round(testing.matmul_tflops(m, m, m, med), 1)}
            del sa_, sb_, sc_
        extra["bf16_gemm_sweep"] = sweep
        for name, build in secondary_workloads(lib, dev, n).items():
            fn, work, kind, info, iters = build()
            ms = quick(fn, iters=iters, warmup=max(5, iters // 3))
            if kind == "flops":
                rec = {"ms": round(ms, 4), "tflops": round(work / ms / 1e9, 1), "frac_of_peak": round(work / ms / 1e9 / PEAK[info["peak"]], 4)}
                if info.get("clock"):
                    rec.update(observed_board_state(fn))
            else:
                rec = {"us": round(ms * 1e3, 2), "gbps": round(work / ms / 1e6, 1), "frac_of_hbm": round(work / ms / 1e6 / HBM_GBPS, 4)}
            if info.get("data"):
                rec["data"] = info["data"]
            extra[name] = rec
            del fn
        # What this board's matrix pipes sustain with nothing but MFMAs of the shapes the GEMMs above are built from, on
        # pseudo-random operands, under the same power limit (triton_amd/power_probe.py over mi355_mfma_burn; 0.4 s per
        # shape): the ceiling that the nominal peaks of `roofline.peak` / `frac_of_peak` do not know about.
        from triton_amd import power_probe

        sampler = power_probe.BoardSampler()
        sink = torch.zeros(4, device=dev, dtype=torch.float32)
        ceiling = {}
        for key, want, ref in (("bf16_16x16x32", "bf16 16x16x32", out["value"]), ("fp8_16x16x128", "fp8 16x16x128", extra.get("fp8_e4m3_gemm_8192", {}).get("tflops")),
                               ("mxfp4_16x16x128", "mxfp4 16x16x128", extra.get("mxfp4_gemm_8192", {}).get("tflops"))):
            name, shape, flop_per_round, _ = next(x for x in power_probe.SHAPES if x[0] == want)
            r = power_probe.burn(lib, sink, stream, shape, flop_per_round, True, 0.4, 1, lib.mi355_query(_lib.Q_CU_COUNT), sampler)
            r["gemm_of_this_ceiling"] = round(ref / r["tflops"], 3) if ref else None
            ceiling[key] = r
        extra["bare_mfma_ceiling_random_operands"] = ceiling
        # A control for the same question from the other side: the same kernels on the same full-size inputs with a
        # QUARTER of the CUs at work (64 persistent programs instead of 256, MI355_GEMM_PROGRAMS / MI355_ATTN_PROGRAMS).
        # The board then stays below its power cap and at its full clock, and the rate per CU at work, as a fraction of
        # the peak per CU, is what the kernel's cycles amount to at the clock the peak is quoted at.  (Fewer CUs also
        # share the caches and the memory among fewer: a control, not a projection of the whole device.)
        quarter = {}
        table = secondary_workloads(lib, dev, n)
        def headline():
            qa = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
            qb = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
            qc = torch.empty(n, n, device=dev, dtype=torch.bfloat16)

            def fn():
                rc = lib.mi355_gemm(qa.data_ptr(), qb.data_ptr(), qc.data_ptr(), n, n, n, n, 1, n, 1, n, 1,
                                    _lib.BF16, _lib.BF16, None, None, 0, stream)
                assert rc == 0, rc

            return fn, flops, "flops", {"peak": "bf16"}, 20
        for key, build in (("bf16_gemm_8192", headline), ("fp8_e4m3_gemm_8192", table["fp8_e4m3_gemm_8192"]),
                           ("mxfp4_gemm_8192", table["mxfp4_gemm_8192"]), ("attn_fwd_causal", table["attn_fwd_causal"])):
            fn, work, _, info, _ = build()
            os.environ["MI355_GEMM_PROGRAMS"] = os.environ["MI355_ATTN_PROGRAMS"] = "64"
            lib.mi355_refresh_env()
            try:
                settle(fn, 0.1)
                _, ms, _ = time_launches(fn, 10, 2)
                rec = {"programs": 64, "ms": round(ms, 4), "tflops": round(work / ms / 1e9, 1),
                       "frac_of_peak_per_cu_at_work": round(work / ms / 1e9 * 4 / PEAK[info["peak"]], 4)}
                rec.update(observed_board_state(fn, 0.5))
            finally:
                del os.environ["MI355_GEMM_PROGRAMS"], os.environ["MI355_ATTN_PROGRAMS"]
                lib.mi355_refresh_env()
            quarter[key] = rec
            del fn
        extra["quarter_of_the_cus_at_full_clock"] = quarter
        out["extra"] = extra

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_gemm()
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
