"""The benchmark harnesses under the environment flags a user may set: every combination must run to its report (a
missing name for a layout, an operand form a flag switches off, a figure that only exists for int8 operands)."""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

FLAGS = [
    {},
    {"BSI_KEY_IMAGE_TILED": "1"},
    {"BSI_KEY_INT8_IMAGE": "0"},
    {"BSI_KEY_LAYOUT": "canonical"},
    {"BSI_KEY_LAYOUT": "canonical", "BSI_KEY_INT8_IMAGE": "0"},
    {"BSI_DOT_CORE": "valu"},
    {"BSI_FIXED_BITS": "0"},
    {"BSI_FIXED_BITS": "0", "BSI_DECIMAL_MFMA": "0"},
    {"BSI_FIXED_CHUNK_SCALE": "0"},
    {"BSI_FIXED_CLIP_K": "3"},
    {"BSI_FIXED_BITS_QUERIES": "8", "BSI_FIXED_BITS_KEYS": "5"},
    {"BSI_FIXED_BITS_QUERIES": "12", "BSI_FIXED_BITS_KEYS": "10"},
    {"BSI_PROFILE": "1"},
]


@pytest.fixture()
def flags(monkeypatch, request):
    from bsipytorch_amd import bsi_ops

    for k in list(os.environ):
        if k.startswith("BSI_"):
            monkeypatch.delenv(k)
    for k, v in request.param.items():
        monkeypatch.setenv(k, v)
    bsi_ops._reset_flag_cache()
    yield request.param
    bsi_ops._reset_flag_cache()


@pytest.mark.parametrize("flags", FLAGS, indirect=True, ids=lambda f: ",".join(f"{k[4:]}={v}" for k, v in f.items()) or "default")
def test_dot_micro_benchmark_reports(flags):
    from bsipytorch_amd.benchmarks import benchmark_dot_kernel_micro as micro

    for kw in ({}, {"relu": True}, {"outliers": True}, {"use_ints8": False}):
        r = micro.run(48, 80, 1024, 2, 0.5, 1, 2, 123, "auto", **kw)
        assert r["avg_dot_us"] > 0 and r["Q"] == 48 and r["R"] == 80 and isinstance(r["layout"], str)


@pytest.mark.parametrize("flags", [{}, {"BSI_KEY_IMAGE_TILED": "1"}, {"BSI_FIXED_BITS": "0"}, {"BSI_DOT_CORE": "valu"}],
                         indirect=True, ids=["default", "tiled-image", "decimal", "valu"])
def test_layer_sweep_reports(flags, monkeypatch):
    from bsipytorch_amd.benchmarks import benchmark_layer_sweep as sweep

    monkeypatch.setitem(sweep.MODELS, "tiny", (256, 1024))
    rows = sweep.run("tiny", Qs=(1, 40), iters=2, warmup=1)
    assert len(rows) == 6 and all(r["avg_dot_us"] > 0 for r in rows)
    torch.cuda.synchronize()


@pytest.mark.parametrize("flags,options", [({}, {}), ({}, {"fuse_qkv": True}), ({}, {"quantize_lm_head": True, "dense": True}),
                                           ({"BSI_FIXED_BITS": "0"}, {}), ({"BSI_QUERY_CACHE": "0"}, {}),
                                           ({"BSI_KEY_IMAGE_TILED": "1"}, {"fuse_qkv": True})],
                         indirect=["flags"], ids=["default", "fuse", "lm_head+dense", "decimal", "no-cache", "tiled-image+fuse"])
def test_prefill_benchmark_reports(flags, options, monkeypatch):
    """benchmark_opt_prefill on a two-layer model of OPT's shape: eager, replayed graph (checked against eager by the
    benchmark itself) and the per-call profile; decimal mode has no graph leg."""
    from bsipytorch_amd.benchmarks import benchmark_opt_prefill as prefill

    monkeypatch.setitem(prefill.SHAPES, "tiny", (2, 256, 4, 1024, 512))
    kw = dict(dense=False)
    kw.update(options)
    r = prefill.run("tiny", seq_len=64, batch=1, iters=2, warmup=1, **kw)
    assert r["num_bsi_layers"] == (13 if options.get("quantize_lm_head") else 12) and r["bsi_fwd_ms"] > 0
    if flags.get("BSI_FIXED_BITS") == "0":
        assert r["bsi_graph_fwd_ms"] is None
    else:
        assert r["graph_replays_match_eager"] is True and r["bsi_graph_fwd_ms"] > 0
    assert r["dot_ms_per_prefill"] > 0


@pytest.mark.parametrize("flags", [{}, {"BSI_FIXED_BITS": "0"}, {"BSI_KEY_INT8_IMAGE": "0"}], indirect=True,
                         ids=["default", "decimal", "no-image"])
def test_apples_to_apples_and_dense_benchmarks_report(flags):
    from bsipytorch_amd.benchmarks import benchmark_apples_to_apples_bsi as apples
    from bsipytorch_amd.benchmarks import benchmark_dense_matmul_micro as dense

    r = apples.run_modes(["kernel_only", "linear_e2e"], 40, 72, 1024, 2, 0.5, 1, 2, 123, "fp16")
    assert set(r) == {"kernel_only", "linear_e2e"} and all(v["bsi_ms"] > 0 and v["torch_ms"] > 0 for v in r.values())
    for dt in ("fp16", "bf16", "fp32"):
        assert dense.run(40, 72, 1024, dt, 1, 2)
