"""What this board's matrix pipes sustain under its power limit: `python -m triton_amd.power_probe`.

Runs the library's bare MFMA loops (`mi355_mfma_burn`: one MFMA shape issued back to back from registers on every
SIMD, no memory traffic) for a sustained period each - 16-bit 32x32x16 and 16x16x32, fp8 32x32x64 and 16x16x128,
fp4 likewise, and the block-scaled forms of the fp4 shapes; pseudo-random and constant operands - and prints, per leg, the rate from device events next to the
board power and shader clock that the driver reports meanwhile (hwmon power1_average / power1_input and
power1_cap, pp_dpm_sclk).  The nominal peaks (2.5 / 5 / 10.1 PFLOP/s) assume 2.4 GHz on every CU; under the
power cap the clock settles where the kernel's energy per flop puts it, and the figures printed here are what a
GEMM built from that MFMA shape can approach on the board at hand.  The measurement counterpart of the
reference's peak helper (python/triton/testing.py:404-426), which computes a rate from a clock argument.
"""
from __future__ import annotations

import argparse
import glob
import json
import os
import re
import sys
import threading
import time

SHAPES = [  # (name, enum of include/mi355_kernels.h, flop per wave and round, nominal peak TFLOP/s)
    ("bf16 32x32x16", 0, 8 * 32768, 2500.0),
    ("bf16 16x16x32", 1, 16 * 16384, 2500.0),
    ("fp8 32x32x64", 2, 8 * 131072, 5000.0),
    ("fp8 16x16x128", 3, 16 * 65536, 5000.0),
    ("fp4 32x32x64", 4, 8 * 131072, 10100.0),
    ("fp4 16x16x128", 5, 16 * 65536, 10100.0),
    ("mxfp4 32x32x64", 6, 8 * 131072, 10100.0),
    ("mxfp4 16x16x128", 7, 16 * 65536, 10100.0),
]


class BoardSampler:
    """Samples watts and shader clock from the driver's files every 10 ms on a host thread."""

    def __init__(self):
        hw = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*"))
        self.power = [q for d in hw for q in (os.path.join(d, "power1_average"), os.path.join(d, "power1_input")) if os.path.exists(q)]
        self.clock = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
        self.cap = None
        for d in hw:
            try:
                self.cap = max(self.cap or 0.0, int(open(os.path.join(d, "power1_cap")).read()) / 1e6)
            except (OSError, ValueError):
                pass
        self.watts, self.mhz, self._stop, self._thread = [], [], False, None

    def _poll(self):
        while not self._stop:
            for path in self.power[:1]:
                try:
                    self.watts.append(int(open(path).read()) / 1e6)
                except (OSError, ValueError):
                    pass
            for path in self.clock[:1]:
                try:
                    m = re.search(r"(\d+)\s*Mhz\s*\*", open(path).read(), re.I)
                    if m:
                        self.mhz.append(int(m.group(1)))
                except OSError:
                    pass
            time.sleep(0.01)

    def __enter__(self):
        self.watts, self.mhz, self._stop = [], [], False
        self._thread = threading.Thread(target=self._poll)
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        self._thread.join()

    @staticmethod
    def _median_tail(xs):
        tail = sorted(xs[len(xs) // 4:])
        return float(tail[len(tail) // 2]) if tail else None

    def result(self):
        return {"power_w": self._median_tail(self.watts), "sclk_mhz": self._median_tail(self.mhz), "power_cap_w": self.cap}


def burn(lib, sink, stream, shape, flop_per_round, random_operands, seconds, waves, cus, sampler):
    """`seconds` of back-to-back launches of one shape; rate from device events over the launches after the first
    quarter of the period (the clocks settle within tens of milliseconds)."""
    import torch

    iters = 4000                                                   # a launch of 4000 rounds runs 2-3 ms
    flop = float(cus) * 4 * waves * iters * flop_per_round

    def launch():
        rc = lib.mi355_mfma_burn(sink.data_ptr(), shape, int(random_operands), iters, waves, stream)
        assert rc == 0, rc

    launch()
    torch.cuda.synchronize()
    events = [torch.cuda.Event(enable_timing=True)]
    events[0].record()
    t0 = time.perf_counter()
    with sampler:
        while time.perf_counter() - t0 < seconds:
            for _ in range(4):
                launch()
                events.append(torch.cuda.Event(enable_timing=True))
                events[-1].record()
            events[-1].synchronize()
    ms = [events[i].elapsed_time(events[i + 1]) for i in range(len(events) - 1)]
    ms = sorted(ms[len(ms) // 4:])
    med = ms[len(ms) // 2]
    return {"tflops": round(flop / med / 1e9, 1), "ms_per_launch": round(med, 4), **sampler.result()}


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--seconds", type=float, default=1.5, help="sustained period per leg")
    ap.add_argument("--waves", type=int, default=1, choices=(1, 2), help="waves per SIMD")
    ap.add_argument("--json", action="store_true", help="print one JSON object instead of the table")
    args = ap.parse_args(argv)

    import torch

    from . import _lib

    assert torch.cuda.is_available(), "power_probe needs the GPU"
    lib = _lib.load()
    cus = lib.mi355_query(_lib.Q_CU_COUNT)
    sink = torch.zeros(4, device="cuda", dtype=torch.float32)
    stream = torch.cuda.current_stream().cuda_stream
    sampler = BoardSampler()
    rows = []
    for name, shape, flop_per_round, peak in SHAPES:
        for random_operands in (True, False):
            r = burn(lib, sink, stream, shape, flop_per_round, random_operands, args.seconds, args.waves, cus, sampler)
            r.update(shape=name, operands="random" if random_operands else "constant", frac_of_nominal_peak=round(r["tflops"] / peak, 3))
            rows.append(r)
    if args.json:
        print(json.dumps({"cus": cus, "waves_per_simd": args.waves, "seconds_per_leg": args.seconds, "legs": rows}))
        return 0
    print(f"{torch.cuda.get_device_name(0)}, {cus} CUs, {args.waves} wave(s) per SIMD, {args.seconds} s per leg, power cap {sampler.cap} W")
    print(f"{'MFMA shape':<16}{'operands':<10}{'TFLOP/s':>9}{'of nominal':>12}{'watts':>8}{'sclk MHz':>10}")
    for r in rows:
        w = "-" if r["power_w"] is None else f"{r['power_w']:.0f}"
        c = "-" if r["sclk_mhz"] is None else f"{r['sclk_mhz']:.0f}"
        print(f"{r['shape']:<16}{r['operands']:<10}{r['tflops']:>9.1f}{r['frac_of_nominal_peak']:>12.3f}{w:>8}{c:>10}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
