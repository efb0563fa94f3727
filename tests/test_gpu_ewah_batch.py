"""Query batches kept as EWAH streams (the batched hybrid form) through bsi_hip_dot_ewah_batch: the decode runs in
the dot's load stage -- inside the few-rows kernel up to 32 rows on tiled planes, as the call's first launch above --
and the result must be what the same dot gives on the verbatim planes: integer accumulators and fp32 outputs
bit-identical to the oracle.  Streams come from the oracle's encoder (so the test does not depend on the GPU
encoder) and, through the ``bsi_ops`` mirror, from the GPU encoder, which must write the same words."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from bsipytorch_amd import _lib

    return _lib


@pytest.fixture()
def ops(monkeypatch):
    from bsipytorch_amd import bsi_ops

    for k in list(os.environ):
        if k.startswith("BSI_"):
            monkeypatch.delenv(k)
    bsi_ops._reset_flag_cache()
    yield bsi_ops
    bsi_ops._reset_flag_cache()


def _dev(a):
    if a.dtype == np.uint64:
        a = a.view(np.int64)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _st():
    return torch.cuda.current_stream().cuda_stream


def _queries(Q, d, seed, kind):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((Q, d)).astype(np.float32)
    if kind == "relu":
        x = np.maximum(x, 0)
    elif kind == "small":          # high planes are pure sign extension: long runs of all-zero and all-one words
        x *= np.float32(0.05)
    elif kind == "sparse":         # mostly exact zeros: every plane compresses
        x[rng.random((Q, d)) < 0.97] = 0.0
    if Q > 2 and d >= 512:
        x[1, :256] = 0.0           # an all-zero chunk
        x[2, 300] = 655.35         # an outlier: one chunk with a large scale
    return x


def _streams(oracle, words, thr):
    """Oracle-encoded streams of planes [Q, Sa, W]: (stream words, offsets, lengths, flags), stream q * Sa + s."""
    Q, Sa, W = words.shape
    flat = words.reshape(Q * Sa, W)
    flags = oracle.compress_flags(flat, thr)
    stream, off, lens = oracle.ewah_encode(flat, flags)
    return stream, off, lens, flags


def _key_operand(hip, kb, R, W, layout):
    L = hip.lib
    chunks = (W + 3) // 4
    B = _dev(kb["words"])
    if layout == 2:
        Bi = torch.full((R, chunks * 256), 77, dtype=torch.int8, device="cuda")
        hip.check(L.bsi_hip_planes_to_int8(B.data_ptr(), R, 6, W, Bi.data_ptr(), _st()), "key image")
        return Bi
    if layout == 1:
        Bt = torch.full((((R + 15) // 16) * chunks * 6 * 64,), -1, dtype=torch.int64, device="cuda")
        hip.check(L.bsi_hip_tile_key_planes(B.data_ptr(), R, 6, W, Bt.data_ptr(), _st()), "tile")
        return Bt
    return B


def _run(hip, oracle, Q, R, d, kind, thr, layout, want_ints, with_bias, seed):
    L = hip.lib
    x = _queries(Q, d, seed, kind)
    rng = np.random.default_rng(seed + 7)
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    k[R // 2] *= 50.0
    qb, kb = oracle.build_queries(x), oracle.build_keys(k)
    W, chunks = (d + 63) // 64, (d + 255) // 256
    want_i, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    stream, off, lens, flags = _streams(oracle, qb["words"], thr)
    comp = _dev(stream if stream.size else np.zeros(1, dtype=np.uint64))
    offd, lend = _dev(off), _dev(lens)
    scales = _dev(qb["scales"])
    stride = chunks if qb["chunk_scale"] else 1
    B, Bw = _key_operand(hip, kb, R, W, layout), _dev(kb["slice_weights"])
    bias = torch.from_numpy(rng.standard_normal(R).astype(np.float32)).cuda() if with_bias else None
    R_total = R + 3
    out = torch.full((Q, R_total), float("nan"), dtype=torch.float32, device="cuda")
    ints = torch.full((Q, R, chunks), -7, dtype=torch.int32, device="cuda") if want_ints else None
    nbytes = int(L.bsi_hip_dot_ewah_batch_workspace_bytes(Q, W))
    ws = torch.full((max(nbytes, 16),), 0x55, dtype=torch.uint8, device="cuda")
    hip.check(L.bsi_hip_dot_ewah_batch(comp.data_ptr(), offd.data_ptr(), lend.data_ptr(), 7, W, scales.data_ptr(), stride,
                                       B.data_ptr(), layout, Bw.data_ptr(), 6, R, Q, float(np.float32(1e-4)), R_total,
                                       bias.data_ptr() if bias is not None else None, out.data_ptr(),
                                       ints.data_ptr() if ints is not None else None, ws.data_ptr(), nbytes, _st()),
              "bsi_hip_dot_ewah_batch")
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    expect = want + bias.cpu().numpy()[None, :] if with_bias else want
    np.testing.assert_array_equal(got[:, :R], expect)
    assert np.isnan(got[:, R:]).all()                      # columns past R are the caller's
    if want_ints:
        np.testing.assert_array_equal(ints.cpu().numpy(), want_i)
    return flags.reshape(Q, 7), lens.reshape(Q, 7)


# (Q, R, d): one query, a ragged group, exactly one and two groups of 16, one past each; tile edges of the int8 kernel
SHAPES = [(1, 200, 4096), (5, 33, 256), (16, 75, 2048), (17, 50, 1024), (32, 40, 2048), (33, 129, 512),
          (130, 70, 2048), (9, 20, 700), (3, 24, 8192), (12, 30, 16640)]


@pytest.mark.parametrize("Q,R,d", SHAPES)
@pytest.mark.parametrize("kind,thr", [("relu", 0.5), ("small", 1.0), ("sparse", 0.5), ("randn", 0.0)])
def test_ewah_batch_dot_matches_oracle(hip, oracle, Q, R, d, kind, thr):
    for layout in (1, 2, 0):     # tiled planes (inline decode up to 32 rows), int8 image, canonical planes
        flags, lens = _run(hip, oracle, Q, R, d, kind, thr, layout, want_ints=(layout != 2 or Q > 40), with_bias=(layout == 2),
                           seed=Q * 3 + d)
    if kind == "relu":
        assert (lens[:, 6] == 1).all() and flags[:, 6].all()       # the empty sign plane: one marker, skipped by the decoder
    if thr == 0.0:   # only a slice of one value throughout (density exactly 0 or 1) is still flagged: one marker
        assert ((flags == 0) & (lens == (d + 63) // 64 + 1) | (flags == 1) & (lens == 1)).all()


@pytest.mark.parametrize("outliers", [False, True])
def test_ewah_batch_at_the_fc2_like_shape(ops, oracle, outliers):
    """Q512 x R2048 x D8192 with ReLU queries at compress_threshold 0.5, built and encoded on the GPU.  On the plain
    distribution the sign plane of every row is one marker and nothing else compresses (with per-chunk scales plane 5
    ends up about 3 % dense, far above the 0.54 % cut).  With one large activation per chunk in the even rows and two
    in the odd rows the high planes sit on both sides of the cut: plane 5 is run/literal coded in the even rows
    (three clean words in four) and verbatim in the odd ones, plane 4 is empty.  Either way the whole output equals
    the oracle's, with and without the bias in the epilogue, and the verbatim batch's dot."""
    torch.manual_seed(123)
    Q, R, D = 512, 2048, 8192
    X = torch.relu(torch.randn(Q, D))
    if outliers:
        X[:, 7::256] = 12.0
        X[1::2, 100::256] = 12.0
    K = torch.randn(R, D) * 0.02
    bias = torch.randn(R)
    kcap, *_ = ops.build_bsi_keys_cuda(K, 2, 0.5)
    hb = ops.build_bsi_queries_cuda_batch_hybrid(X.cuda(), 2, 0.5)
    flags, lens = hb.flags.view(Q, 7).cpu().numpy(), hb.comp_len.view(Q, 7).cpu().numpy()
    assert flags[:, 6].all() and (lens[:, 6] == 1).all()              # no negative value: one marker per row
    if outliers:
        assert flags[0::2, 5].all() and not flags[1::2, 5].any()      # rows on both sides of the density cut
        assert (lens[0::2, 5] == 65).all() and (lens[1::2, 5] == 129).all()     # 32 literals + 33 markers against 1 + 128
        assert flags[:, 4].all() and (lens[:, 4] <= 3).all()          # a plane that is empty but for a stray bit, between two used ones
        assert hb.mem_bytes < hb.verbatim_bytes * 5.6 / 7
    else:
        assert not flags[:, :6].any()
        assert hb.verbatim_bytes * 5.9 / 7 < hb.mem_bytes < hb.verbatim_bytes * 6.2 / 7   # a seventh saved, less markers and offsets
    # the GPU encoder writes the oracle's streams
    qb = oracle.build_queries(X.numpy())
    stream, off, olens, oflags = _streams(oracle, qb["words"], 0.5)
    np.testing.assert_array_equal(hb.comp_words.cpu().numpy().view(np.uint64), stream)
    np.testing.assert_array_equal(hb.comp_len.cpu().numpy(), olens)
    kb = oracle.build_keys(K.numpy())
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    out = ops.batch_dot_product_multiquery_cuda_batch_caps(hb, kcap)[0]
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    with_bias = ops.batch_dot_product_multiquery_cuda_batch_caps(hb, kcap, bias.cuda())[0]
    np.testing.assert_array_equal(with_bias.cpu().numpy(), want + bias.numpy()[None, :])
    verbatim = ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.5)
    assert torch.equal(ops.batch_dot_product_multiquery_cuda_batch_caps(verbatim, kcap)[0], out)


@pytest.mark.parametrize("Q", [1, 4, 16, 32])
def test_ewah_batch_few_rows_through_ops(ops, oracle, Q):
    """Decode-sized batches against an OPT-6.7B-shaped layer (4096 x 4096): the inline-decode kernel."""
    torch.manual_seed(Q)
    R, D = 4096, 4096
    X = torch.relu(torch.randn(Q, D))
    K = torch.randn(R, D) * 0.02
    kcap, *_ = ops.build_bsi_keys_cuda(K, 2, 0.5)
    hb = ops.build_bsi_queries_cuda_batch_hybrid(X.cuda(), 2, 0.5)
    out = ops.batch_dot_product_multiquery_cuda_batch_caps(hb, kcap)[0]
    qb, kb = oracle.build_queries(X.numpy()), oracle.build_keys(K.numpy())
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    np.testing.assert_array_equal(out.cpu().numpy(), want)


def test_ewah_batch_argument_checks(hip):
    L = hip.lib
    t = torch.zeros(64, dtype=torch.int64, device="cuda")
    args = lambda Q, ws_bytes, Sa=7, stride=8: (t.data_ptr(), t.data_ptr(), t.data_ptr(), Sa, 32, t.data_ptr(), stride,
                                                t.data_ptr(), 2, t.data_ptr(), 6, 64, Q, 1.0, 64, None, t.data_ptr(), None,
                                                t.data_ptr(), ws_bytes, _st())
    assert L.bsi_hip_dot_ewah_batch(*args(64, 16)) == 1 and b"workspace" in L.bsi_hip_last_error()
    assert L.bsi_hip_dot_ewah_batch(*args(64, 1 << 20, Sa=9)) == 1
    assert L.bsi_hip_dot_ewah_batch(*args(64, 1 << 20, stride=3)) == 1 and b"stride" in L.bsi_hip_last_error()
    assert L.bsi_hip_dot_ewah_batch(*args(0, 0)) == 0
    assert L.bsi_hip_dot_ewah_batch_workspace_bytes(512, 128) == 512 * 8192
