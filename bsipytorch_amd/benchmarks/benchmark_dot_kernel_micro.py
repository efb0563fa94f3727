"""Microbenchmark of the BSI dot kernel on one GPU (same flags as the reference's
``bsi_ops/benchmarks/benchmark_dot_kernel_micro.py``, plus the core, key layout and input shaping
of the FC1/FC2-like configurations).

    python -m bsipytorch_amd.benchmarks.benchmark_dot_kernel_micro --Q 512 --R 8192 --D 2048 --outliers
    python -m bsipytorch_amd.benchmarks.benchmark_dot_kernel_micro --Q 512 --R 2048 --D 8192 --relu

The kernel time is measured with HIP events around ``iters`` back-to-back launches on the launch
stream; no environment flag is needed (the reference prints zeros unless BSI_PROFILE=1).
"""
import argparse
import ctypes
import json

import torch

from bsipytorch_amd import _lib, bsi_ops


def run(Q, R, D, decimal_places=2, compress_threshold=0.5, warmup=10, iters=50, seed=123, core="auto",
        key_sigma=0.02, outliers=False, relu=False, use_ints8=True, report_stats=False, image_fill="built"):
    torch.manual_seed(seed)
    K = torch.randn(R, D, dtype=torch.float32) * key_sigma
    X = torch.randn(Q, D, dtype=torch.float32)
    if outliers:
        X[:, torch.randperm(D)[: max(1, D // 1000)]] *= 20.0
    if relu:
        X = torch.relu(X)
    kcap, key_bytes, _, _, W = bsi_ops.build_bsi_keys_cuda(K, decimal_places, float(compress_threshold))
    qcap = bsi_ops.build_bsi_queries_cuda_batch_packed(X.cuda(), decimal_places, float(compress_threshold))
    if report_stats:
        print("[Keys]", bsi_ops.bsi_keys_cuda_stats(kcap))
    if image_fill != "built":
        _refill_images(qcap, kcap, image_fill)
    chunks = (W + 3) // 4
    if not (qcap.fixed and kcap.fixed):
        return _run_weighted(qcap, kcap, Q, R, D, W, key_bytes, warmup, iters)
    if qcap.chunk_scales is not None:
        scales, stride = qcap.chunk_scales, chunks
    else:
        scales, stride = qcap.row_scales, 1
    code = {"auto": _lib.CORE_AUTO, "mfma": _lib.CORE_MFMA, "valu": _lib.CORE_VALU}[core]
    use_ints8 = use_ints8 and qcap.ints8 is not None  # operands wider than 8 bits have no int8 image
    out = torch.empty((Q, R), dtype=torch.float32, device="cuda")
    ws_bytes = 0 if use_ints8 else int(_lib.lib.bsi_hip_dot_workspace_bytes(Q, W, code))
    ws = torch.empty((max(ws_bytes, 16),), dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    kptr, klayout = bsi_ops.key_operand(kcap, Q, qcap.Sa, code)
    bsi_ops.attach_split_scratch()  # as every dot through bsi_ops does: the D-split route, where the launcher picks it
    tile, segments = ctypes.c_int(0), ctypes.c_int(0)
    _lib.check(_lib.lib.bsi_hip_dot_split_plan(R, Q, W, ctypes.byref(tile), ctypes.byref(segments)), "bsi_hip_dot_split_plan")
    args = (qcap.words.data_ptr(), qcap.ints8.data_ptr() if use_ints8 else None, scales.data_ptr(), stride, qcap.Sa, W,
            kptr, klayout, kcap.slice_weights.data_ptr(), kcap.Sb, R, Q, 1.0 / 10.0 ** (2 * decimal_places),
            R, out.data_ptr(), code, ws.data_ptr(), ws_bytes)
    us = ctypes.c_float(0.0)
    if warmup > 0:
        _lib.check(_lib.lib.bsi_hip_dot_timed(*args, warmup, ctypes.byref(us), st), "warmup")
    _lib.check(_lib.lib.bsi_hip_dot_timed(*args, iters, ctypes.byref(us), st), "timed")
    t = float(us.value) * 1e-6
    bit_ops = 2.0 * qcap.Sa * kcap.Sb * Q * R * D
    alg_bytes = Q * qcap.Sa * W * 8 + Q * chunks * 4 + R * kcap.Sb * W * 8 + R * 4 + Q * R * 4
    return {"Q": Q, "R": R, "D": D, "core": core, "layout": {0: "canonical", 1: "tiled16", 2: "int8 image", 3: "int8 image in 64-row tiles"}[klayout],
            "i8_tile": tile.value if klayout >= 2 else None, "d_split_segments": segments.value if klayout >= 2 else None,
            "avg_dot_us": t * 1e6, "dot_q_us": t * 1e6 / Q, "dot_s_ns": t * 1e9 / (Q * R),
            "effective_bitop_TOPS": bit_ops / t / 1e12, "int8_TOPS": 2.0 * Q * R * D / t / 1e12,
            "algorithmic_GBps": alg_bytes / t / 1e9, "key_plane_GBps": key_bytes / t / 1e9, "iters": iters}


def _refill_images(qcap, kcap, fill):
    """Overwrite the int8 images the matrix-core kernel reads, for timing only (the output is then not the dot of
    the inputs).  The kernel does the same instructions on any data, so a change of its time with the data is the
    shader clock following the power the operands draw: "zero" toggles nothing, "random" is uniform bytes,
    "magnitude" keeps the built values without their signs (no runs of one-bits from sign extension)."""
    if qcap.ints8 is None or kcap.ints8 is None:
        raise RuntimeError("--image_fill needs fixed-bit operands with int8 images")
    for cap in (qcap, kcap):
        if fill == "zero":
            cap.ints8.zero_()
        elif fill == "random":
            cap.ints8.copy_(torch.randint(-128, 128, cap.ints8.shape, dtype=torch.int8, device=cap.ints8.device))
        elif fill == "magnitude":
            cap.ints8.copy_(cap.ints8.abs())
        else:
            raise ValueError(fill)


def _run_weighted(qcap, kcap, Q, R, D, W, key_bytes, warmup, iters):
    """Decimal-mode operands (BSI_FIXED_BITS*=0): the weighted-slice dot, timed by device events over `iters` calls."""
    for _ in range(max(warmup, 1)):
        bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    e1.record()
    e1.synchronize()
    t = e0.elapsed_time(e1) * 1e-3 / iters
    bit_ops = 2.0 * qcap.Sa * kcap.Sb * Q * R * D
    alg_bytes = Q * qcap.Sa * W * 8 + R * kcap.Sb * W * 8 + (Q * qcap.Sa + R * kcap.Sb) * 4 + Q * R * 4
    on_mfma = (getattr(qcap, "digits8", None) is not None or (qcap.fixed and qcap.ints8 is not None)) and \
              (getattr(kcap, "digits8", None) is not None or (kcap.fixed and kcap.ints8 is not None))
    return {"Q": Q, "R": R, "D": D, "core": "int8 digits on MFMA" if on_mfma else "weighted popcount (VALU)",
            "layout": "canonical" if kcap.layout == 0 else "tiled16",
            "Sa": qcap.Sa, "Sb": kcap.Sb, "avg_dot_us": t * 1e6, "dot_q_us": t * 1e6 / Q, "dot_s_ns": t * 1e9 / (Q * R),
            "effective_bitop_TOPS": bit_ops / t / 1e12, "popcount_word_ops_per_s": qcap.Sa * kcap.Sb * Q * R * W / t,
            "algorithmic_GBps": alg_bytes / t / 1e9, "key_plane_GBps": key_bytes / t / 1e9, "iters": iters}


def main() -> None:
    p = argparse.ArgumentParser(description="Microbench BSI dot kernel (HIP, gfx950)")
    p.add_argument("--Q", type=int, default=128)
    p.add_argument("--R", type=int, default=256)
    p.add_argument("--D", type=int, default=2048)
    p.add_argument("--decimal_places", type=int, default=2)
    p.add_argument("--compress_threshold", type=float, default=0.5)
    p.add_argument("--warmup", type=int, default=5)
    p.add_argument("--iters", type=int, default=20)
    p.add_argument("--seed", type=int, default=123)
    p.add_argument("--core", default="auto", choices=["auto", "mfma", "valu"])
    p.add_argument("--key_sigma", type=float, default=0.02)
    p.add_argument("--outliers", action="store_true", help="scale 0.1%% of the query columns by 20")
    p.add_argument("--relu", action="store_true", help="ReLU the queries (about half exact zeros)")
    p.add_argument("--planes_only", action="store_true", help="do not hand the builder's int8 queries to the dot")
    p.add_argument("--report_stats", action="store_true")
    p.add_argument("--i8_tile", type=int, default=0, choices=[0, 128, 1284, 12864, 64, 6432],
                   help="force a tile of the int8-image kernel (1284: 128 x 128 on four MFMA waves of 64 x 64); 0 = automatic")
    p.add_argument("--split", type=int, default=0,
                   help="D-split of the int8-image kernel: 0 = by the launcher's cost model, 1 = never, n >= 2 = n segments "
                        "per output tile (on --i8_tile 128 or 12864)")
    p.add_argument("--image_fill", default="built", choices=["built", "zero", "random", "magnitude"],
                   help="timing only: overwrite the int8 images (the clock follows the power the data draws)")
    a = p.parse_args()
    if not torch.cuda.is_available():
        raise RuntimeError("a GPU is required for this microbench")
    _lib.check(_lib.lib.bsi_hip_set_option(_lib.OPT_I8_TILE, a.i8_tile), "bsi_hip_set_option")
    _lib.check(_lib.lib.bsi_hip_set_option(_lib.OPT_I8_SPLIT, a.split), "bsi_hip_set_option")
    r = run(a.Q, a.R, a.D, a.decimal_places, a.compress_threshold, a.warmup, a.iters, a.seed, a.core, a.key_sigma,
            a.outliers, a.relu, not a.planes_only, a.report_stats, a.image_fill)
    print(f"[Microbench] Q={a.Q} R={a.R} D={a.D} iters={a.iters} core={r['core']} layout={r['layout']}")
    print(f"[Kernel] avg_dot_ms={r['avg_dot_us'] / 1e3:.4f}  dot_q_us={r['dot_q_us']:.3f}  dot_s_ns={r['dot_s_ns']:.4f}")
    print(json.dumps(r))


if __name__ == "__main__":
    main()
