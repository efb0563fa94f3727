"""Slice-count (Sb) and word-count (W) statistics of the BSI keysets of a quantised model.

Counterpart of ``bsi_ops/benchmarks/collect_bsi_shape_stats.py`` of the reference, on the locally built
OPT-shaped model of ``benchmark_opt_prefill`` (random weights; no download).  In fixed-bit mode every key has
the configured slice count; with ``BSI_FIXED_BITS_KEYS=0`` (decimal mode) the count follows the weights.

    python -m bsipytorch_amd.benchmarks.collect_bsi_shape_stats --model opt-125m
"""
from __future__ import annotations

import argparse
from collections import Counter

import torch

from bsipytorch_amd import bsi_ops, linear
from bsipytorch_amd.benchmarks.benchmark_opt_prefill import SHAPES, build_model


def collect(model) -> dict:
    sb_hist, w_hist, rows = Counter(), Counter(), []
    for name, module in model.named_modules():
        if isinstance(module, linear.BSIQuantizedLinear):
            stats = bsi_ops.bsi_keys_cuda_stats(module._bsi_keys_cuda)
            w_hist[int(stats["W"])] += 1
            for sb, cnt in stats["Sb_counts"].items():
                sb_hist[int(sb)] += int(cnt)
            rows.append((name, int(stats["W"]), dict(stats["Sb_counts"])))
    return {"W": dict(w_hist), "Sb": dict(sb_hist), "layers": rows}


def main() -> None:
    ap = argparse.ArgumentParser(description="Collect BSI shape stats (Sb/W) per layer")
    ap.add_argument("--model", default="opt-125m", choices=sorted(SHAPES))
    ap.add_argument("--decimal_places", type=int, default=2)
    ap.add_argument("--compress_threshold", type=float, default=0.5)
    ap.add_argument("--scope", default="all", choices=["all", "attention", "mlp"])
    ap.add_argument("--seed", type=int, default=123)
    a = ap.parse_args()
    if not torch.cuda.is_available():
        raise RuntimeError("a GPU is required: the keysets are built on the device")
    model = build_model(a.model, a.seed, "cuda")
    linear.quantize_model_bsi(model, decimalPlaces=a.decimal_places, scope=a.scope,
                              compress_threshold=a.compress_threshold, verbose=False)
    res = collect(model)
    print("=== W (words per slice) distribution across layers ===")
    for w, cnt in sorted(res["W"].items()):
        print(f"W={w}: {cnt} layers")
    print("\n=== Sb (slices per key) distribution across all keys ===")
    for sb, cnt in sorted(res["Sb"].items()):
        print(f"Sb={sb}: {cnt} keys")
    print("\n=== Per-layer breakdown (name, W, Sb_counts) ===")
    for name, w, sb_counts in res["layers"]:
        print(f"{name}: W={w}, Sb_counts={sb_counts}")


if __name__ == "__main__":
    main()
