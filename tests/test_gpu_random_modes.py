"""Seeded sweeps of the two operand forms beside fixed76 planes, on drawn shapes, value ranges and thresholds, each held
to the oracle bit for bit: decimal mode (slice counts from the data, weighted-slice dot on either route) and query
batches kept as EWAH streams (decoded in the dot's load stage; every compress threshold, dense to all-zero inputs)."""
import os
import numpy as np
import pytest
import torch

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


@pytest.fixture(scope="module")
def oracle():
    from oracle import bsi_oracle
    return bsi_oracle


def host_u64(t):
    return t.cpu().numpy().view(np.uint64)


@pytest.mark.parametrize("seed", range(32))
def test_decimal_mode_on_drawn_shapes(ops, oracle, monkeypatch, seed):
    rng = np.random.default_rng(9000 + seed)
    monkeypatch.setenv("BSI_FIXED_BITS", "0")
    ops._reset_flag_cache()
    Q = int(rng.choice([1, 2, 5, 16, 33, 64, 130]))
    R = int(rng.choice([1, 7, 16, 40, 64, 100, 200]))
    D = int(rng.choice([1, 5, 64, 100, 256, 300, 512, 1024, 2048]))
    dec = int(rng.choice([0, 1, 2, 3]))
    xs = float(rng.choice([0.01, 1.0, 30.0]))
    ks = float(rng.choice([0.02, 1.0, 10.0]))
    x = (rng.standard_normal((Q, D)) * xs).astype(np.float32)
    k = (rng.standard_normal((R, D)) * ks).astype(np.float32)
    if rng.random() < 0.3:
        x[:] = np.maximum(x, 0)
    if rng.random() < 0.2:
        x[0, :] = 0
    a, b = oracle.build_decimal(x, dec), oracle.build_decimal(k, dec)
    want = oracle.dot_weighted(a["words"], a["slice_weights"], b["words"], b["slice_weights"], oracle.scale_inv(dec, dec))
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), dec, 0.2)
    qcap = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(x).cuda(), dec, 0.2)
    assert qcap.Sa == a["S"]
    np.testing.assert_array_equal(host_u64(qcap.words), a["words"])
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("seed", range(32))
def test_ewah_stream_batches_on_drawn_shapes(ops, oracle, seed):
    rng = np.random.default_rng(12000 + seed)
    Q = int(rng.choice([1, 2, 5, 16, 17, 32, 33, 64, 130, 300]))
    R = int(rng.choice([1, 16, 40, 64, 100, 200, 260]))
    D = int(rng.choice([256, 512, 768, 1024, 2048, 2304, 4096]))
    thr = float(rng.choice([0.0, 0.2, 0.5, 0.9, 1.0]))
    kind = str(rng.choice(["randn", "relu", "small", "sparse", "zero"]))
    x = rng.standard_normal((Q, D)).astype(np.float32)
    if kind == "relu":
        x = np.maximum(x, 0)
    elif kind == "small":
        x *= np.float32(0.05)
    elif kind == "sparse":
        x[rng.random((Q, D)) < 0.97] = 0.0
    elif kind == "zero":
        x[:] = 0
    k = (rng.standard_normal((R, D)) * 0.02).astype(np.float32)
    qb, kb = oracle.build_queries(x), oracle.build_keys(k)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.5)
    hb = ops.build_bsi_queries_cuda_batch_hybrid(torch.from_numpy(x).cuda(), 2, thr)
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(hb, kcap)
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))
    bias = torch.from_numpy(rng.standard_normal(R).astype(np.float32)).cuda()
    outb, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(hb, kcap, bias)
    np.testing.assert_array_equal(outb.cpu().numpy(), want + bias.cpu().numpy()[None, :])
    if Q == 1:
        h, *_ = ops.build_bsi_query_cuda_hybrid(torch.from_numpy(x[0]).cuda(), 2, thr)
        o1, *_ = ops.batch_dot_product_multiquery_cuda_caps([h], kcap)
        # the one-query hybrid form carries a row scale (no chunk scales): its own oracle value
        ints, shifts, scales = oracle.quantize_fixed(x, 2, 7, False)
        _, w1 = oracle.dot_fixed(oracle.pack(ints, 7), scales, kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
        np.testing.assert_array_equal(o1.cpu().numpy().view(np.uint32), w1.view(np.uint32))
