"""Dense ``X @ K.T`` on the same shapes as the BSI dot microbenchmark, as the dense baseline
(flags of the reference's ``bsi_ops/benchmarks/benchmark_dense_matmul_micro.py``).

    python -m bsipytorch_amd.benchmarks.benchmark_dense_matmul_micro --Q 512 --R 8192 --D 2048 --dtype fp32
"""
import argparse
import json
import time

import torch

_DTYPES = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}


def run(Q, R, D, dtype="fp16", warmup=10, iters=50, seed=123, allow_tf32=False):
    torch.manual_seed(seed)
    torch.backends.cuda.matmul.allow_tf32 = bool(allow_tf32)
    dt = _DTYPES[dtype]
    x = torch.randn(Q, D, dtype=torch.float32).to("cuda", dt)
    w = (torch.randn(R, D, dtype=torch.float32) * 0.02).to("cuda", dt)
    out = torch.empty((Q, R), dtype=dt, device="cuda")
    for _ in range(warmup):
        torch.matmul(x, w.T, out=out)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        torch.matmul(x, w.T, out=out)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / iters
    return {"Q": Q, "R": R, "D": D, "dtype": dtype, "avg_mm_us": ms * 1e3, "mm_q_us": ms * 1e3 / Q,
            "mm_s_ns": ms * 1e6 / (Q * R), "TFLOPs": 2.0 * Q * R * D / (ms * 1e-3) / 1e12, "iters": iters}


def main() -> None:
    p = argparse.ArgumentParser(description="Dense matmul microbench (baseline for the BSI dot)")
    p.add_argument("--Q", type=int, default=512)
    p.add_argument("--R", type=int, default=8192)
    p.add_argument("--D", type=int, default=2048)
    p.add_argument("--dtype", type=str, default="fp16", choices=sorted(_DTYPES))
    p.add_argument("--allow_tf32", action="store_true")
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--iters", type=int, default=50)
    p.add_argument("--seed", type=int, default=123)
    a = p.parse_args()
    if not torch.cuda.is_available():
        raise RuntimeError("a GPU is required for this microbench")
    t0 = time.perf_counter()
    r = run(a.Q, a.R, a.D, a.dtype, a.warmup, a.iters, a.seed, a.allow_tf32)
    print(f"[Dense Microbench] Q={a.Q} R={a.R} D={a.D} dtype={a.dtype} iters={a.iters}")
    print(f"[Kernel] avg_mm_ms={r['avg_mm_us'] / 1e3:.3f}  mm_q_us={r['mm_q_us']:.3f}  mm_s_ns={r['mm_s_ns']:.3f}")
    print(f"[Wall] total_elapsed_s={time.perf_counter() - t0:.3f}")
    print(json.dumps(r))


if __name__ == "__main__":
    main()
