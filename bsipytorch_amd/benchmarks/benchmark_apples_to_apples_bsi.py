"""BSI against a dense matmul on equal footing, two of the modes of the reference's
``bsi_ops/benchmarks/benchmark_apples_to_apples_bsi.py``:

* ``kernel_only``: the dot on prebuilt query and key planes vs ``torch.matmul`` on resident operands;
* ``linear_e2e``: query build + dot (what a BSI-linear forward costs) vs the same matmul.

(The reference's third mode, ``model_e2e``, shells out to its LAMBADA harness, which needs downloads;
``benchmark_opt_prefill`` covers the model-level comparison on random weights.)

    python -m bsipytorch_amd.benchmarks.benchmark_apples_to_apples_bsi --Q 512 --R 8192 --D 2048 --torch_dtype fp32
"""
import argparse
import json
from typing import Callable, Dict, List

import torch

from bsipytorch_amd import bsi_ops

_DTYPES = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}


def _time_cuda_ms(fn: Callable[[], None], warmup: int, iters: int) -> float:
    for _ in range(max(0, warmup)):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def _row(name: str, ms: float, q: int, r: int) -> None:
    print(f"{name:22s} avg_ms={ms:.4f}  us_per_query={ms * 1e3 / q:.3f}  ns_per_scalar={ms * 1e6 / (q * r):.4f}")


def run_modes(modes: List[str], Q: int, R: int, D: int, decimal_places: int, threshold: float, warmup: int, iters: int,
              seed: int, torch_dtype: str) -> Dict[str, Dict[str, float]]:
    torch.manual_seed(seed)
    k_cpu = torch.randn(R, D, dtype=torch.float32) * 0.02
    q_fp32 = torch.randn(Q, D, dtype=torch.float32, device="cuda")
    dt = _DTYPES[torch_dtype]
    w = k_cpu.to("cuda", dt)
    x = q_fp32.to(dt)
    keys, *_ = bsi_ops.build_bsi_keys_cuda(k_cpu, decimal_places, threshold)
    res: Dict[str, Dict[str, float]] = {}
    t_torch = _time_cuda_ms(lambda: torch.matmul(x, w.T), warmup, iters)
    if "kernel_only" in modes:
        print("\n[Mode] kernel_only")
        qcap = bsi_ops.build_bsi_queries_cuda_batch_packed(q_fp32, decimal_places, threshold)
        t_bsi = _time_cuda_ms(lambda: bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, keys), warmup, iters)
        _row("bsi_dot", t_bsi, Q, R)
        _row(f"torch_matmul_{torch_dtype}", t_torch, Q, R)
        print(f"speedup_vs_torch = {t_torch / t_bsi:.4f}x")
        res["kernel_only"] = {"bsi_ms": t_bsi, "torch_ms": t_torch, "speedup_vs_torch": t_torch / t_bsi}
    if "linear_e2e" in modes:
        print("\n[Mode] linear_e2e")

        def bsi_linear() -> None:
            qc = bsi_ops.build_bsi_queries_cuda_batch_packed(q_fp32, decimal_places, threshold)
            bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(qc, keys)

        t_bsi = _time_cuda_ms(bsi_linear, warmup, iters)
        _row("bsi_build_plus_dot", t_bsi, Q, R)
        _row(f"torch_matmul_{torch_dtype}", t_torch, Q, R)
        print(f"speedup_vs_torch = {t_torch / t_bsi:.4f}x")
        res["linear_e2e"] = {"bsi_ms": t_bsi, "torch_ms": t_torch, "speedup_vs_torch": t_torch / t_bsi}
    return res


def main() -> None:
    p = argparse.ArgumentParser(description="BSI vs dense matmul, kernel-only and build+dot")
    p.add_argument("--modes", type=str, default="kernel_only,linear_e2e")
    p.add_argument("--Q", type=int, default=128)
    p.add_argument("--R", type=int, default=256)
    p.add_argument("--D", type=int, default=2048)
    p.add_argument("--decimal_places", type=int, default=2)
    p.add_argument("--compress_threshold", type=float, default=0.5)
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--iters", type=int, default=50)
    p.add_argument("--seed", type=int, default=123)
    p.add_argument("--torch_dtype", type=str, default="fp16", choices=sorted(_DTYPES))
    a = p.parse_args()
    if not torch.cuda.is_available():
        raise RuntimeError("a GPU is required for this benchmark")
    modes = [m.strip() for m in a.modes.split(",") if m.strip()]
    for m in modes:
        if m not in ("kernel_only", "linear_e2e"):
            raise SystemExit(f"unsupported mode {m!r} (kernel_only, linear_e2e)")
    print("[Config]")
    print(f"  modes={modes}  shape=(Q={a.Q}, R={a.R}, D={a.D})  decimal_places={a.decimal_places}  "
          f"compress_threshold={a.compress_threshold}  warmup={a.warmup}  iters={a.iters}  torch_dtype={a.torch_dtype}")
    res = run_modes(modes, a.Q, a.R, a.D, a.decimal_places, float(a.compress_threshold), a.warmup, a.iters, a.seed,
                    a.torch_dtype)
    print("\n[Summary]")
    print(json.dumps(res))


if __name__ == "__main__":
    main()
