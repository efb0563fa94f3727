"""A seeded sweep of the int8-image dot over ragged shapes, through the C ABI, bit for bit against the oracle.

Every case draws Q, R, the chunk count, the row stride of the output, the tile, the store kind, the image layout and
whether a bias is added, so that tile edges, padded outputs, whole-line and element stores and both key-image layouts
meet in combinations the hand-picked cases of test_gpu_parity.py do not list.  The draws are fixed by the seeds below.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TILES = (0, 128, 1284, 12864, 64, 6432)


@pytest.fixture(scope="module")
def hip():
    from bsipytorch_amd import _lib
    return _lib


@pytest.fixture(scope="module")
def oracle():
    from oracle import bsi_oracle
    return bsi_oracle


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _stream():
    return torch.cuda.current_stream().cuda_stream


@pytest.mark.parametrize("seed", range(24))
def test_int8_image_dot_on_drawn_shapes(hip, oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    Q = int(rng.choice([33, 48, 64, 70, 127, 128, 129, 200, 256, 300]))
    R = int(rng.choice([17, 64, 100, 128, 130, 192, 255, 256, 288, 416, 513]))
    chunks = int(rng.choice([1, 2, 3, 4, 5, 8, 9]))
    d, W = chunks * 256, chunks * 4
    pad = int(rng.choice([0, 0, 5, 32, 96]))          # output row stride R + pad: 0 and 32 / 96 keep lines aligned
    tile = int(rng.choice(TILES))
    stores = int(rng.choice([0, 1, 2]))
    image_tiled = bool(rng.integers(0, 2))
    with_bias = bool(rng.integers(0, 2))
    kind = str(rng.choice(["randn", "relu", "outliers"]))
    print(f"seed {seed}: Q{Q} R{R} D{d} pad{pad} tile{tile} stores{stores} tiled{image_tiled} bias{with_bias} {kind}", flush=True)

    x = rng.standard_normal((Q, d)).astype(np.float32)
    if kind == "relu":
        x = np.maximum(x, 0)
    elif kind == "outliers":
        x[:, rng.integers(0, d, size=3)] *= 20
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    qb, kb = oracle.build_queries(x, 2, 7), oracle.build_keys(k, 2, 6)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    bias = rng.standard_normal(R).astype(np.float32)
    if with_bias:
        want = want + bias[None, :]

    L = hip.lib
    A, scales, Bc, Bw, bd = _dev(qb["words"]), _dev(qb["scales"]), _dev(kb["words"]), _dev(kb["slice_weights"]), _dev(bias)
    a8 = torch.zeros((Q, chunks * 256), dtype=torch.int8, device="cuda")
    hip.check(L.bsi_hip_planes_to_int8(A.data_ptr(), Q, 7, W, a8.data_ptr(), _stream()), "query image")
    if image_tiled:
        B = torch.full((int(L.bsi_hip_int8_tiled_bytes(R, W)),), 77, dtype=torch.int8, device="cuda")
        hip.check(L.bsi_hip_planes_to_int8_tiled(Bc.data_ptr(), R, 6, W, B.data_ptr(), _stream()), "key image")
        layout = 3
    else:
        B = torch.full((R, chunks * 256), 77, dtype=torch.int8, device="cuda")
        hip.check(L.bsi_hip_planes_to_int8(Bc.data_ptr(), R, 6, W, B.data_ptr(), _stream()), "key image")
        layout = 2
    R_total = R + pad
    out = torch.full((Q, R_total), float("nan"), dtype=torch.float32, device="cuda")
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, tile), "opt")
    hip.check(L.bsi_hip_set_option(hip.OPT_OUTPUT_STORES, stores), "opt")
    try:
        if with_bias:
            hip.check(L.bsi_hip_dot_bias(A.data_ptr(), a8.data_ptr(), scales.data_ptr(), chunks, 7, W, B.data_ptr(), layout,
                                         Bw.data_ptr(), 6, R, Q, float(np.float32(1e-4)), R_total, bd.data_ptr(),
                                         out.data_ptr(), 2, None, 0, _stream()), "dot_bias")
        else:
            hip.check(L.bsi_hip_dot(A.data_ptr(), a8.data_ptr(), scales.data_ptr(), chunks, 7, W, B.data_ptr(), layout,
                                    Bw.data_ptr(), 6, R, Q, float(np.float32(1e-4)), R_total, out.data_ptr(), None, 2, None,
                                    0, _stream()), "dot")
        torch.cuda.synchronize()
    finally:
        hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, 0), "opt")
        hip.check(L.bsi_hip_set_option(hip.OPT_OUTPUT_STORES, 0), "opt")
    got = out.cpu().numpy()
    np.testing.assert_array_equal(got[:, :R], want)
    assert np.isnan(got[:, R:]).all()
