"""Where the int8-image chunk-scale dot spends its time, from wall-clock stamps inside the kernel.

Needs the timeline build of the library (`make -C bsipytorch_amd/csrc TIMELINE=1`), selected with
`BSI_HIP_LIBRARY=bsipytorch_amd/libbsi_hip_timeline.so`; the ordinary build carries no stamps and
`bsi_hip_timeline_read` says so.  For every shape the dot is launched back to back (HIP events give the period per
launch), then the stamps of the last launch are read: per workgroup, lane 0 of one MFMA wave and of one loader wave
note the 100 MHz wall clock when they enter, when the first stage load is issued, when three stages are issued, when
the first stage is in LDS, when the chunk loop is done and when the outputs have left the wave.  Printed relative to
the earliest stamp of the launch, as min / median / max over the workgroups.  The differences between two stamps of
one workgroup are the reliable part; stamps of different workgroups are compared on the assumption that all XCDs read
the same clock, and the clock is taken at its nominal 100 MHz.

    BSI_HIP_LIBRARY=bsipytorch_amd/libbsi_hip_timeline.so python -m bsipytorch_amd.benchmarks.kernel_timeline
"""
from __future__ import annotations

import argparse
import ctypes
import json

import numpy as np
import torch

from bsipytorch_amd import _lib
from bsipytorch_amd.benchmarks import benchmark_dot_kernel_micro as micro

STAMPS = ("mfma wave entered", "first stage in LDS", "chunk loop done", "outputs stored", "loader wave entered",
          "loader wave done", "first stage load issued", "three stages issued")
ORDER = (4, 0, 6, 7, 1, 5, 2, 3)  # the order things happen in


def timeline(Q: int, R: int, D: int, iters: int = 50, warmup: int = 10) -> dict:
    wgs = 8192
    buf = (ctypes.c_ulonglong * (wgs * 8))()
    _lib.check(_lib.lib.bsi_hip_timeline_read(buf, wgs), "bsi_hip_timeline_read")  # clears what earlier launches left
    res = micro.run(Q, R, D, 2, 0.5, warmup, iters, 123, "mfma", outliers=(D == 2048))
    cbuf = (ctypes.c_ulonglong * (wgs * 8))()
    _lib.check(_lib.lib.bsi_hip_timeline_read_cycles(cbuf, wgs), "bsi_hip_timeline_read_cycles")  # before the read that clears
    _lib.check(_lib.lib.bsi_hip_timeline_read(buf, wgs), "bsi_hip_timeline_read")
    t = np.frombuffer(buf, dtype=np.uint64).reshape(wgs, 8).astype(np.int64)
    cyc = np.frombuffer(cbuf, dtype=np.uint64).reshape(wgs, 8).astype(np.int64)[t[:, 0] > 0]
    live = t[t[:, 0] > 0]  # the workgroups of this shape's grid
    base = min(live[:, 0].min(), live[:, 4].min())
    us = (live - base) / 100.0
    out = {"Q": Q, "R": R, "D": D, "us_per_launch_by_events": round(res["avg_dot_us"], 2), "workgroups": int(len(us)),
           "stamps_us": {}}
    for i in ORDER:
        c = us[:, i]
        out["stamps_us"][STAMPS[i]] = {"min": round(float(c.min()), 2), "median": round(float(np.median(c)), 2),
                                      "max": round(float(c.max()), 2)}
    halves = 2 * ((D + 255) // 256)
    loop = float(np.median(us[:, 2] - us[:, 1]))
    out["per_workgroup_median_us"] = {
        "entry_to_first_issue": round(float(np.median(us[:, 6] - us[:, 4])), 2),
        "issuing_three_stages": round(float(np.median(us[:, 7] - us[:, 6])), 2),
        "chunk_loop": round(loop, 2),
        "chunk_loop_per_half_chunk": round(loop / halves, 3),
        "output_stores": round(float(np.median(us[:, 3] - us[:, 2])), 2),
    }
    # the shader clock's own counter over the chunk loop: cycles per half-chunk (512 is what the MFMAs of a 128 x 128
    # tile need, and what 32 KiB take at 64 bytes per clock), and the clock the GPU held there
    loop_cycles = (cyc[:, 2] - cyc[:, 1]).astype(np.float64)
    loop_ticks = (live[:, 2] - live[:, 1]).astype(np.float64)
    out["per_workgroup_median_us"]["chunk_loop_cycles_per_half_chunk"] = round(float(np.median(loop_cycles)) / halves, 1)
    out["per_workgroup_median_us"]["shader_clock_GHz_in_the_loop"] = round(float(np.median(loop_cycles / (loop_ticks / 100.0))) / 1e3, 3)
    out["in_kernel_us"] = round(float(us[:, 3].max()), 2)
    out["between_launches_us"] = round(out["us_per_launch_by_events"] - out["in_kernel_us"], 2)
    return out


def main() -> None:
    p = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--shapes", nargs="*", default=["512x8192x2048", "512x8192x8192", "512x2048x8192", "512x2048x2048"],
                   help="QxRxD")
    p.add_argument("--iters", type=int, default=50)
    p.add_argument("--warmup", type=int, default=10,
                   help="untimed launches before the timed ones; several thousand bring the shader clock to the state "
                        "it holds under sustained load (about 35 ms of work from an idle GPU)")
    args = p.parse_args()
    for sh in args.shapes:
        Q, R, D = (int(v) for v in sh.lower().split("x"))
        print(json.dumps(timeline(Q, R, D, args.iters, args.warmup)), flush=True)


if __name__ == "__main__":
    main()
