#!/usr/bin/env python3
"""Benchmark of the gfx950 GGUF k-quant matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extra] [--no-cpu]

One "step" is one pass of the hot path over one batch of synthetic input: the
fused q8_1 decode GEMV of a Q4_K 17408x5120 weight at batch 1 (the shape the
headline metric is quoted on).  Inputs are resident in HBM before the timed
region; the weight rotates over enough distinct copies (> 256 MB) that the
Infinity Cache cannot hold it, so the figure is an HBM figure.  The timed
region is bracketed by device synchronisations and, for the roofline figure,
by HIP events recorded on the launch stream.

Prints ONE JSON line.  `value` is algorithmic bytes per step / time per step.
The host side is torch-free (ctypes HIP binding).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0        # dense int8 MFMA, published
METRIC = "Q4_K decode GEMV GB/s (% HBM peak); MMQ prefill int8 TOPS (% MFMA peak)"
GGML = {"q8_0": 8, "q4_k": 12, "q6_k": 14}
BLOCK = {"q8_0": (32, 34), "q4_k": (256, 144), "q6_k": (256, 210)}
MALL_BYTES = 256 << 20


def gemv_bytes(quant: str, rows: int, k: int, n: int, act_bytes: int = 4) -> int:
    """Algorithmic bytes of one GEMV: weights once, activations in, float32 out."""
    bs, tb = BLOCK[quant]
    return n * (k // bs) * tb + rows * k * act_bytes + rows * n * 4


class Harness:
    def __init__(self):
        from hipengine_amd.core import memory
        from hipengine_amd.core.build import load_library
        from hipengine_amd.core.hip import get_hip_runtime

        self.memory = memory
        self.rt = get_hip_runtime()
        if self.rt.device_count() < 1:
            raise SystemExit("bench.py needs one HIP device (MI355X)")
        self.rt.set_device(0)
        load_library()   # raises if the library is not built: there is no CPU fallback
        self.ev0, self.ev1 = self.rt.event_create(), self.rt.event_create()

    def time_launches(self, launch, steps: int, warmup: int):
        """(wall seconds per step, HIP-event seconds per step) over exactly `steps` launches."""
        for i in range(warmup):
            launch(i)
        self.rt.device_synchronize()
        t0 = time.perf_counter()
        self.rt.event_record(self.ev0, 0)
        for i in range(steps):
            launch(i)
        self.rt.event_record(self.ev1, 0)
        self.rt.device_synchronize()
        wall = (time.perf_counter() - t0) / steps
        ev = self.rt.event_elapsed_time_ms(self.ev0, self.ev1) * 1e-3 / steps
        return wall, ev

    def gemv_case(self, quant: str, rows: int, k: int, n: int, steps: int, warmup: int, seed: int = 0):
        from hipengine_amd.kernels.hip_gfx950.quant import gguf_q8_1_gemv as G
        from hipengine_amd.synthetic import synthetic_blocks

        w = synthetic_blocks(GGML[quant], n, k, seed=seed)
        copies = max(2, -(-2 * MALL_BYTES // w.nbytes))        # working set >= 2x the Infinity Cache
        free, _ = self.rt.mem_get_info()
        copies = int(max(1, min(copies, (free // 2) // max(w.nbytes, 1))))
        wbufs = [self.memory.to_device(w, runtime=self.rt) for _ in range(copies)]
        x = np.random.default_rng(seed + 1).standard_normal((rows, k)).astype(np.float32)
        dx = self.memory.to_device(x, runtime=self.rt)
        dout = self.memory.malloc(rows * n * 4, runtime=self.rt)
        fn = G.FUSED[(quant, "f32", "f32")]
        wall, ev = self.time_launches(lambda i: fn(dx.ptr, wbufs[i % copies].ptr, dout.ptr, rows, k, n), steps, warmup)
        for buf in (*wbufs, dx, dout):
            self.memory.free(buf)
        return {"bytes": gemv_bytes(quant, rows, k, n), "wall_s": wall, "event_s": ev, "copies": copies,
                "weight_host": w, "x_host": x}


def cpu_baseline(w: np.ndarray, x: np.ndarray, nbytes: int) -> dict:
    """The reference CPU backend path (dequantize the whole weight to float32, then a
    float32 matmul; hipengine/kernels/cpu_reference/ops.py:466-484) as restated by
    the oracle, timed on the host cores: 1 warmup + 3 repeats, median."""
    from oracle import gguf_oracle as O

    times = []
    for rep in range(4):
        t0 = time.perf_counter()
        O.gguf_quant_gemv(x, w, O.GGML_Q4_K)
        if rep:
            times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {"value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": os.cpu_count() or 1, "kind": "port",
            "ms": round(med * 1e3, 2),
            "sample": "full workload (Q4_K 17408x5120 b1), NumPy dequantize + float32 matmul, "
                      "1 warmup + 3 repeats, median"}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary shapes")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this path is single-GPU (run with --gpus 1)")

    h = Harness()
    k, n = 5120, 17408
    main_case = h.gemv_case("q4_k", 1, k, n, args.steps, args.warmup)
    gbs = main_case["bytes"] / main_case["wall_s"] / 1e9
    achieved = main_case["bytes"] / main_case["event_s"] / 1e9

    extra = {}
    if not args.no_extra:
        steps = max(20, args.steps // 5)
        for name, (quant, rows, kk, nn) in {
            "q4_k_17408x5120_b2": ("q4_k", 2, 5120, 17408),
            "q8_0_5120x5120_b1": ("q8_0", 1, 5120, 5120),
            "q6_k_5120x17408_b1": ("q6_k", 1, 17408, 5120),
            "q6_k_151936x5120_b1": ("q6_k", 1, 5120, 151936),
        }.items():
            c = h.gemv_case(quant, rows, kk, nn, steps, max(5, args.warmup // 5))
            extra[name] = {"us": round(c["event_s"] * 1e6, 2), "GB/s": round(c["bytes"] / c["event_s"] / 1e9, 1),
                           "frac_hbm": round(c["bytes"] / c["event_s"] / 1e9 / HBM_PEAK_GBS, 4), "copies": c["copies"]}

    result = {
        "metric": METRIC,
        "value": round(gbs, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_case["wall_s"] * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 dot / f32 combine",
        "data": "synthetic",
        "config": {"workload": "Q4_K 17408x5120 decode GEMV, batch 1, f32 activations quantized to q8_1 in-kernel",
                   "weight_copies_rotated": main_case["copies"], "bytes_per_step": main_case["bytes"]},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel_us": round(main_case["event_s"] * 1e6, 3)},
        "cpu_baseline": None if args.no_cpu else cpu_baseline(main_case["weight_host"], main_case["x_host"],
                                                               main_case["bytes"]),
        "extra": extra,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
