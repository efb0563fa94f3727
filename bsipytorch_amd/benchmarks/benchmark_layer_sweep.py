"""Per-layer BSI dot sweep over model-shaped key matrices and token counts.

Default: the OPT-6.7B linear shapes (attention 4096x4096, fc1 16384x4096, fc2 4096x16384) at
Q = 1, 16, 128, 512 query rows.  Small Q is the decode regime, bound by reading the packed key
planes from HBM once (0.75 byte per weight); the sweep prints that bandwidth next to the compute
figures.  One JSON line per (layer, Q).

    python -m bsipytorch_amd.benchmarks.benchmark_layer_sweep [--model opt-6.7b] [--Q 1 16 128 512]
"""
import argparse
import json

import torch

from bsipytorch_amd.benchmarks import benchmark_dot_kernel_micro as micro

HBM_PEAK_GBS = 8000.0
MFMA_I8_PEAK_TOPS = 5000.0

MODELS = {  # hidden, ffn
    "opt-1.3b": (2048, 8192),
    "opt-6.7b": (4096, 16384),
}


def layer_shapes(model: str):
    hidden, ffn = MODELS[model]
    return [("attn_proj", hidden, hidden), ("fc1", ffn, hidden), ("fc2", hidden, ffn)]


def run(model="opt-6.7b", Qs=(1, 16, 128, 512), core="auto", iters=50, warmup=10, seed=123):
    rows = []
    for name, R, D in layer_shapes(model):
        for Q in Qs:
            r = micro.run(Q, R, D, 2, 0.5, warmup, iters, seed, core)
            r["layer"] = name
            r["model"] = model
            r["key_plane_frac_of_hbm_peak"] = r["key_plane_GBps"] / HBM_PEAK_GBS
            r["algorithmic_frac_of_hbm_peak"] = r["algorithmic_GBps"] / HBM_PEAK_GBS
            if "int8_TOPS" in r:  # absent in decimal mode, whose operands are not int8
                r["int8_frac_of_mfma_peak"] = r["int8_TOPS"] / MFMA_I8_PEAK_TOPS
            rows.append(r)
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", default="opt-6.7b", choices=sorted(MODELS))
    ap.add_argument("--Q", type=int, nargs="+", default=[1, 16, 128, 512])
    ap.add_argument("--core", default="auto", choices=["auto", "mfma", "valu"])
    ap.add_argument("--iters", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--seed", type=int, default=123)
    a = ap.parse_args()
    if not torch.cuda.is_available():
        raise RuntimeError("a GPU is required for this sweep")
    for r in run(a.model, tuple(a.Q), a.core, a.iters, a.warmup, a.seed):
        print(json.dumps(r), flush=True)


if __name__ == "__main__":
    main()
