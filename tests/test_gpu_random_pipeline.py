"""A seeded sweep of the whole path -- builder, the dot the dispatcher picks, and the BSI-linear layer with its bias --
over drawn row counts, key counts, widths, activation dtypes and value ranges, bit for bit against the oracle.  The
layer is quantised while it lives on the CPU and fed device activations (so its bias stays on the host), or moved to the
device first: every combination of few rows / many rows, fp32 / half precision and host / device bias takes another
route through the layer."""
import os

import numpy as np
import pytest
import torch
import torch.nn as nn

pytestmark = pytest.mark.gpu


@pytest.fixture()
def ops(monkeypatch):
    from bsipytorch_amd import bsi_ops

    for k in list(os.environ):
        if k.startswith("BSI_"):
            monkeypatch.delenv(k)
    bsi_ops._reset_flag_cache()
    yield bsi_ops
    bsi_ops._reset_flag_cache()


@pytest.mark.parametrize("seed", range(40))
def test_pipeline_and_layer_on_drawn_shapes(ops, oracle, seed):
    from bsipytorch_amd.linear import BSIQuantizedLinear, forget_shared_builds

    rng = np.random.default_rng(5000 + seed)
    Q = int(rng.choice([1, 2, 3, 4, 5, 15, 16, 17, 31, 32, 33, 40, 64, 100, 128, 130, 260]))
    R = int(rng.choice([1, 15, 16, 17, 63, 64, 65, 100, 128, 200, 256, 300, 520]))
    D = int(rng.choice([64, 192, 256, 320, 512, 700, 768, 1024, 1280, 2048, 2304, 4096]))
    dt = [torch.float32, torch.float16, torch.bfloat16][int(rng.integers(0, 3))]
    kind = str(rng.choice(["randn", "relu", "outliers", "tiny", "big"]))
    layer_on_device = bool(rng.integers(0, 2))
    print(f"seed {seed}: Q{Q} R{R} D{D} {dt} {kind} layer_on_device={layer_on_device}", flush=True)
    x = rng.standard_normal((Q, D)).astype(np.float32)
    if kind == "relu":
        x = np.maximum(x, 0)
    elif kind == "outliers":
        x[:, rng.integers(0, D, size=2)] *= 30
    elif kind == "tiny":
        x *= 1e-3
    elif kind == "big":
        x *= 1e4
    k = (rng.standard_normal((R, D)) * float(rng.choice([0.02, 1.0, 50.0]))).astype(np.float32)
    xt = torch.from_numpy(x).to(dt)
    x = xt.float().numpy()  # what the builder sees
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.5)
    qcap = ops.build_bsi_queries_cuda_batch_packed(xt.cuda(), 2, 0.5)
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    qb, kb = oracle.build_queries(x), oracle.build_keys(k)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))

    lin = nn.Linear(D, R, bias=True)
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy(k))
        lin.bias.copy_(torch.from_numpy(rng.standard_normal(R).astype(np.float32)))
    layer = BSIQuantizedLinear(lin, decimalPlaces=2, compress_threshold=0.5)
    if layer_on_device:
        layer.cuda()
    assert layer.bias.is_cuda == layer_on_device
    y = layer(xt.cuda())
    assert y.dtype == dt and tuple(y.shape) == (Q, R) and y.is_cuda
    bias = lin.bias.detach()
    # fp32: out + bias in float32; half precision: the scores are cast first, then the cast bias is added
    want_y = torch.from_numpy(want + bias.numpy()[None, :]) if dt == torch.float32 else torch.from_numpy(want).to(dt) + bias.to(dt)
    assert torch.equal(y.cpu(), want_y)
    forget_shared_builds()
