"""A seeded sweep over the environment flags the `bsi_ops` mirror reads -- clipping, chunk or row scales, core, key
layout and int8 image, the one-call and few-rows layer paths, shared query builds, profiling, fp32 queries -- on drawn
shapes, dtypes and value ranges: builder + dot through both query forms, and the BSI-linear layer with its bias, each
held to the oracle bit for bit."""
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


@pytest.fixture(scope="module")
def oracle():
    from oracle import bsi_oracle
    return bsi_oracle


@pytest.mark.parametrize("seed", range(48))
def test_drawn_flags_shapes_and_dtypes(ops, oracle, monkeypatch, seed):
    from bsipytorch_amd.linear import BSIQuantizedLinear, forget_shared_builds
    rng = np.random.default_rng(40000 + seed)
    flags = {}
    clip = float(rng.choice([0.0, 0.0, 2.5, 6.0]))
    if clip:
        flags["BSI_FIXED_CLIP_K"] = str(clip)
    chunk_scale = bool(rng.integers(0, 2))
    if not chunk_scale:
        flags["BSI_FIXED_CHUNK_SCALE"] = "0"
    for name, choices in (("BSI_DOT_CORE", ["auto", "mfma", "valu"]), ("BSI_KEY_LAYOUT", ["tiled", "canonical"]),
                          ("BSI_KEY_INT8_IMAGE", ["1", "0"]), ("BSI_KEY_IMAGE_TILED", ["0", "1"]), ("BSI_TC_DOT", ["1", "0"]),
                          ("BSI_FUSED_LINEAR", ["1", "0", "2"]), ("BSI_LINEAR_ONE_CALL", ["1", "0"]), ("BSI_QUERY_PACKED", ["1", "0"]),
                          ("BSI_QUERY_CACHE", ["1", "0"]), ("BSI_PROFILE", ["0", "1"]), ("BSI_QUERY_FP32", ["0", "1"])):
        v = str(rng.choice(choices))
        if v != choices[0]:
            flags[name] = v
    dec = int(rng.choice([0, 1, 2, 2, 3]))
    Q = int(rng.choice([1, 2, 4, 5, 16, 33, 64, 130]))
    R = int(rng.choice([1, 16, 40, 64, 100, 200]))
    D = int(rng.choice([64, 256, 320, 512, 700, 1024, 2048]))
    dt = [torch.float32, torch.float16, torch.bfloat16][int(rng.integers(0, 3))]
    for k_, v_ in flags.items():
        monkeypatch.setenv(k_, v_)
    ops._reset_flag_cache()
    x = (rng.standard_normal((Q, D)) * float(rng.choice([0.1, 1.0, 20.0]))).astype(np.float32)
    if rng.random() < 0.3:
        x[:, rng.integers(0, D, size=2)] *= 40
    k = (rng.standard_normal((R, D)) * float(rng.choice([0.02, 1.0]))).astype(np.float32)
    xt = torch.from_numpy(x).to(dt)
    x = xt.float().numpy()
    W = (D + 63) // 64
    cs = chunk_scale and W % 4 == 0
    ints, shifts, scales = oracle.quantize_fixed(x, dec, 7, cs, clip)
    kints, kshifts, kscales = oracle.quantize_fixed(k, dec, 6, False, clip)
    _, want = oracle.dot_fixed(oracle.pack(ints, 7), scales, oracle.pack(kints, 6), kscales, oracle.scale_inv(dec, dec), want_ints=False)
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), dec, 0.5)
    qcap = ops.build_bsi_queries_cuda_batch_packed(xt.cuda(), dec, 0.5)
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))
    rows = ops.build_bsi_queries_cuda_batch(xt.cuda(), dec, 0.5)
    out2, *_ = ops.batch_dot_product_multiquery_cuda_caps(rows, kcap)
    np.testing.assert_array_equal(out2.cpu().numpy().view(np.uint32), want.view(np.uint32))
    lin = nn.Linear(D, R, bias=True)
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy(k))
    layer = BSIQuantizedLinear(lin, decimalPlaces=dec, compress_threshold=0.5).cuda()
    y = layer(xt.cuda())
    y2 = layer(xt.cuda().clone())
    assert torch.equal(y, y2)
    bias = lin.bias.detach()
    if dt == torch.float32:  # the bias joins the fp32 result; in half precision it is added after the cast
        want_y = torch.from_numpy(want + bias.numpy()[None, :])
    else:
        want_y = torch.from_numpy(want).to(dt) + bias.to(dt)
    assert torch.equal(y.cpu(), want_y), (y.cpu() - want_y).abs().max()
    forget_shared_builds()


@pytest.mark.parametrize("seed", range(32))
def test_drawn_bit_widths_and_flags(ops, oracle, monkeypatch, seed):
    """Other fixed-bit widths (2 to 16 bits, as BSI_FIXED_BITS_QUERIES / _KEYS set them) under drawn flags: builder, dot and
    layer against the oracle built for those widths."""
    from bsipytorch_amd.linear import BSIQuantizedLinear, forget_shared_builds
    rng = np.random.default_rng(60000 + seed)
    bq = int(rng.choice([2, 3, 5, 7, 8, 9, 12, 16]))
    bk = int(rng.choice([2, 4, 6, 8, 9, 13]))
    flags = {"BSI_FIXED_BITS_QUERIES": str(bq), "BSI_FIXED_BITS_KEYS": str(bk)}
    clip = float(rng.choice([0.0, 0.0, 3.0]))
    if clip:
        flags["BSI_FIXED_CLIP_K"] = str(clip)
    chunk_scale = bool(rng.integers(0, 2))
    if not chunk_scale:
        flags["BSI_FIXED_CHUNK_SCALE"] = "0"
    for name, choices in (("BSI_DOT_CORE", ["auto", "mfma", "valu"]), ("BSI_KEY_LAYOUT", ["tiled", "canonical"]),
                          ("BSI_KEY_INT8_IMAGE", ["1", "0"]), ("BSI_KEY_IMAGE_TILED", ["0", "1"]), ("BSI_TC_DOT", ["1", "0"])):
        v = str(rng.choice(choices))
        if v != choices[0]:
            flags[name] = v
    Q = int(rng.choice([1, 3, 16, 33, 64, 130]))
    R = int(rng.choice([1, 16, 40, 100, 200]))
    D = int(rng.choice([64, 256, 512, 700, 1024]))
    for k_, v_ in flags.items():
        monkeypatch.setenv(k_, v_)
    ops._reset_flag_cache()
    x = rng.standard_normal((Q, D)).astype(np.float32)
    k = (rng.standard_normal((R, D)) * 0.05).astype(np.float32)
    W = (D + 63) // 64
    cs = chunk_scale and W % 4 == 0
    ints, shifts, scales = oracle.quantize_fixed(x, 2, bq, cs, clip)
    kints, kshifts, kscales = oracle.quantize_fixed(k, 2, bk, False, clip)
    _, want = oracle.dot_fixed(oracle.pack(ints, bq), scales, oracle.pack(kints, bk), kscales, oracle.scale_inv(2, 2), want_ints=False)
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.5)
    qcap = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(x).cuda(), 2, 0.5)
    try:
        out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    except RuntimeError as e:
        # the matrix cores forced onto operands wider than int8 are refused, never approximated (operands without chunk
        # scales go to the weighted-slice dot, which takes any width, and are compared below like the rest)
        assert flags.get("BSI_DOT_CORE") == "mfma" and (bq > 8 or bk > 8) and "MFMA core needs" in str(e), e
        return
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))
    lin = nn.Linear(D, R, bias=True)
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy(k))
    layer = BSIQuantizedLinear(lin, decimalPlaces=2, compress_threshold=0.5).cuda()
    y = layer(torch.from_numpy(x).cuda())
    np.testing.assert_array_equal(y.cpu().numpy(), want + lin.bias.detach().numpy()[None, :])
    forget_shared_builds()
