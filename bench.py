"""Benchmark of the BSI fixed76 chunk-scale dot on one MI355X.

    python bench.py [--gpus 1] [--steps 50] [--warmup 10] [--core auto|mfma|valu] [--no-cpu]

Workload: the FC1-like configuration (queries fp32 Q=512 x D=2048 ~N(0,1) with 0.1% of the columns
scaled x20, keys fp32 R=8192 x D=2048 ~N(0,0.02), decimal_places=2, compress_threshold=0.5, Sa=7,
Sb=6, chunk scales), synthetic, seed 123.  A step is one dot over the prebuilt query and key planes
(resident in HBM).  Prints ONE JSON line.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
MFMA_I8_PEAK_TOPS = 5000.0     # MI355X published dense int8
Q, R, D = 512, 8192, 2048
# HBM bytes per launch of the dot kernel on this workload, from rocprofv3 FETCH_SIZE and WRITE_SIZE runs scaled by a
# 256 MiB copy (profiles/dot_mfma_i8_kernel_fc1_Q512_R8192_D2048_hbm_traffic.txt); counters cannot be read in-process
MEASURED_TRAFFIC_BYTES = {"mfma": 42466000}
SA, SB = 7, 6


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--core", default="auto", choices=["auto", "mfma", "valu"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a dispatch of known traffic for scaling "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no collectives); run with --gpus 1",
              file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from bsipytorch_amd import _lib, bsi_ops

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)
    torch.manual_seed(123)
    X = torch.randn(Q, D)
    cols = torch.randperm(D)[: max(1, D // 1000)]
    X[:, cols] *= 20.0
    K = torch.randn(R, D) * 0.02

    kcap, key_bytes, _, _, W = bsi_ops.build_bsi_keys_cuda(K, 2, 0.5)
    qcap = bsi_ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.5)
    chunks = W // 4
    core = {"auto": _lib.CORE_AUTO, "mfma": _lib.CORE_MFMA, "valu": _lib.CORE_VALU}[args.core]
    out = torch.empty((Q, R), dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    scale_inv = 1.0 / 10.0 ** 4

    kptr, klayout = bsi_ops.key_operand(kcap, Q, SA, core)

    def dot_args():
        return (qcap.words.data_ptr(), qcap.ints8.data_ptr(), qcap.chunk_scales.data_ptr(), chunks, SA, W,
                kptr, klayout, kcap.slice_weights.data_ptr(), SB, R, Q, scale_inv, R, out.data_ptr())

    def step():
        _lib.check(_lib.lib.bsi_hip_dot(*dot_args(), None, core, None, 0, stream), "bsi_hip_dot")

    if args.calibration_copy:
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall_s = time.perf_counter() - t0
    ms_per_step = wall_s * 1e3 / args.steps

    # kernel duration with HIP events on the launch stream (same K launches, back to back)
    mean_us = ctypes.c_float(0.0)
    _lib.check(_lib.lib.bsi_hip_dot_timed(*dot_args(), core, None, 0, args.steps, ctypes.byref(mean_us), stream),
               "bsi_hip_dot_timed")
    kern_us = float(mean_us.value)

    bit_ops = 2.0 * SA * SB * Q * R * D                  # one AND + one popcount-accumulate per bit-MAC
    int8_ops = 2.0 * Q * R * D                           # the same contraction counted as int8 MACs
    alg_bytes = Q * SA * W * 8 + Q * chunks * 4 + R * SB * W * 8 + R * 4 + Q * R * 4
    used_core = args.core if args.core != "auto" else "mfma"
    hbm_gbs = alg_bytes / (kern_us * 1e-6) / 1e9
    if used_core == "mfma":
        # int8 MFMA contraction: 2*Q*R*D int8 operations per launch against the published dense int8 peak
        roof = {"bound": "mfma", "achieved": int8_ops / (kern_us * 1e-6) / 1e12, "peak": MFMA_I8_PEAK_TOPS,
                "unit": "TFLOP/s", "op": "int8 multiply-add counted as 2 ops (TOP/s)"}
    else:
        # The popcount core is VALU-bound, which the two published roofs do not describe; it is priced
        # against HBM here and against the VALU issue rate in "valu" below.
        roof = {"bound": "hbm", "achieved": hbm_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = MEASURED_TRAFFIC_BYTES.get(used_core)
    roof["kernel_us"] = kern_us
    roof["algorithmic_bytes"] = alg_bytes
    roof["hbm_GBs_algorithmic"] = hbm_gbs
    # one v_and_b32 + one v_bcnt_u32_b32 per 32 bit-MACs; 256 CU x 4 SIMD x 16 lanes x 2.4 GHz lane-ops/s
    valu_peak = 256 * 4 * 16 * 2.4e9 * 32 / 2 / 1e12
    valu = {"achieved_Tbitmac_s": bit_ops / 2 / (kern_us * 1e-6) / 1e12, "peak_Tbitmac_s": valu_peak}
    valu["frac"] = valu["achieved_Tbitmac_s"] / valu_peak

    result = {
        "metric": "bsi_dot_effective_bitop_TOPS@Q512_R8192_D2048",
        "value": bit_ops / (ms_per_step * 1e-3) / 1e12,
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "us_per_call": ms_per_step * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8" if used_core == "mfma" else "u32",
        "dtype_note": "int8 x int8 -> int32 MFMA per 256-element chunk, fp32 fmaf chunk-scale epilogue"
                      if used_core == "mfma" else "u32 and/popcount -> int32 per chunk, fp32 fmaf chunk-scale epilogue",
        "data": "synthetic",
        "config": {"workload": "FC1-like fixed76 chunk-scale dot Q512 R8192 D2048, 0.1% outlier columns x20, dec=2",
                   "core": used_core, "key_layout": {0: "canonical planes", 1: "tiled16 planes", 2: "cached int8 image of the planes"}[klayout],
                   "algorithmic_bytes": alg_bytes, "bit_ops": bit_ops},
        "roofline": roof,
    }
    if used_core == "valu":
        result["valu"] = valu

    # peaks measured on this GPU by the library's probes (a pure v_mfma_i32_16x16x64_i8 loop, a pure
    # v_and/v_bcnt loop, a streaming read of 1 GiB), next to the published figures the roofline uses
    peaks = {"published": {"int8_mfma_TOPS": MFMA_I8_PEAK_TOPS, "hbm_GBs": HBM_PEAK_GBS}}
    v = ctypes.c_double(0.0)
    _lib.check(_lib.lib.bsi_hip_probe_mfma_i8(ctypes.byref(v), stream), "probe_mfma")
    peaks["int8_mfma_TOPS"] = v.value / 1e12
    _lib.check(_lib.lib.bsi_hip_probe_valu_popcount(ctypes.byref(v), stream), "probe_valu")
    peaks["valu_and_bcnt_Tbitmac_s"] = v.value * 32 / 2 / 1e12   # one v_and + one v_bcnt per 32 bit-MACs
    buf = torch.ones(1 << 30, dtype=torch.uint8, device="cuda")
    _lib.check(_lib.lib.bsi_hip_probe_stream_read(buf.data_ptr(), buf.numel(), ctypes.byref(v), stream), "probe_read")
    peaks["stream_read_GBs"] = v.value / 1e9
    del buf
    result["measured_peaks"] = peaks
    result["roofline"]["frac_of_measured_mfma_peak"] = (int8_ops / (kern_us * 1e-6) / 1e12) / peaks["int8_mfma_TOPS"]

    # dense baselines of the same shape on the same GPU (resident operands, same event timing)
    Xd, Kd = X.cuda(), K.cuda()
    dense = {}
    for name, dt in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
        a, b = Xd.to(dt), Kd.to(dt)
        for _ in range(5):
            torch.matmul(a, b.T)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            torch.matmul(a, b.T)
        e1.record()
        torch.cuda.synchronize()
        dense[f"torch_matmul_{name}_us"] = e0.elapsed_time(e1) / 20 * 1e3
    result["dense_baseline"] = dense

    if not args.no_cpu:
        from oracle import bsi_oracle

        A = qcap.words.cpu().numpy().view(np.uint64)
        qs = qcap.chunk_scales.cpu().numpy()
        # canonical key planes for the oracle (rebuilt on the GPU in canonical order, then copied)
        os.environ["BSI_KEY_LAYOUT"] = "canonical"
        bsi_ops._reset_flag_cache()
        kc, *_ = bsi_ops.build_bsi_keys_cuda(K, 2, 0.5)
        B = kc.words.cpu().numpy().view(np.uint64)
        bs = kc.slice_weights[:, 0].contiguous().cpu().numpy()
        reps, t_cpu = 0, 0.0
        while t_cpu < 12.0 and reps < 100:  # a bounded sample: about 12 s of CPU work, whole passes only
            t1 = time.perf_counter()
            _, ref = bsi_oracle.dot_fixed(A, qs, B, bs, np.float32(scale_inv), want_ints=False)
            t_cpu += time.perf_counter() - t1
            reps += 1
        step()
        torch.cuda.synchronize()
        same = bool(np.array_equal(out.cpu().numpy(), ref))
        result["cpu_baseline"] = {"value": bit_ops / (t_cpu / reps) / 1e12, "unit": "TOPS", "cores": bsi_oracle.num_threads(),
                                  "kind": "port", "sample": f"{reps} full passes of the same Q512 R8192 D2048 dot "
                                  f"(oracle popcount form, OpenMP over keys); {t_cpu / reps * 1e3:.1f} ms per pass",
                                  "ms_per_call": t_cpu / reps * 1e3, "gpu_output_bit_identical": same}
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
