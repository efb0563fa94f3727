"""GPU parity: every HIP kernel against the CPU oracle on the same seeded inputs, through the C ABI
(raw entry points) and through the ``bsi_ops`` mirror.  Integer and bit work must be bit-exact; the
fp32 output is compared bit-for-bit as well (same chunk order, fused multiply-add, power-of-two
scales), with the 1e-5 relative tolerance of the specification as the stated bar.
"""
import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")
FP32_RTOL = 1e-5  # stated tolerance for the fp32 outputs; the asserts below ask for exact equality first


@pytest.fixture(scope="module")
def hip():
    assert torch.cuda.is_available(), "these tests need the MI355X"
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


def dev(a: np.ndarray) -> torch.Tensor:
    if a.dtype == np.uint64:
        a = a.view(np.int64)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host_u64(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().numpy().view(np.uint64)


def st():
    return torch.cuda.current_stream().cuda_stream


# ------------------------------------------------------------------ builder


def _inputs(Q, d, seed, kind="randn"):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((Q, d)).astype(np.float32)
    if kind == "outliers":
        cols = rng.permutation(d)[: max(1, d // 1000)]
        x[:, cols] *= 20.0
    elif kind == "relu":
        x = np.maximum(x, 0)
    elif kind == "small":
        x *= np.float32(0.02)
    elif kind == "ties":
        x = (rng.integers(-3000, 3000, size=(Q, d)) / 200.0).astype(np.float32)  # many x.5 after *100
    if Q > 2 and d >= 256:
        x[1, :256] = 0.0       # an all-zero chunk
        x[2, 5] = 655.35       # a large outlier
    return x


@pytest.mark.parametrize("Q,d,kind", [(64, 2048, "randn"), (33, 2048, "outliers"), (17, 8192, "relu"),
                                      (5, 256, "ties"), (9, 700, "randn"), (3, 64, "small"), (4, 1000, "ties")])
@pytest.mark.parametrize("bits,chunk", [(7, True), (6, False), (8, True), (4, False)])
def test_build_fixed_matches_oracle(hip, oracle, Q, d, kind, bits, chunk):
    x = _inputs(Q, d, seed=Q * 7 + d, kind=kind)
    ints, shifts, scales = oracle.quantize_fixed(x, 2, bits, chunk)
    want_words = oracle.pack(ints, bits)
    W = (d + 63) // 64
    chunks = (d + 255) // 256
    xd = dev(x)
    words = torch.zeros((Q, bits, W), dtype=torch.int64, device="cuda")
    sh = torch.zeros(shifts.shape, dtype=torch.int32, device="cuda")
    sc = torch.zeros(scales.shape, dtype=torch.float32, device="cuda")
    i8 = torch.full((Q, chunks * 256), 77, dtype=torch.int8, device="cuda")
    hip.check(hip.lib.bsi_hip_build_fixed(xd.data_ptr(), 0, Q, d, 2, bits, int(chunk), 0.0, words.data_ptr(),
                                          sh.data_ptr(), sc.data_ptr(), i8.data_ptr(), st()), "build")
    torch.cuda.synchronize()
    np.testing.assert_array_equal(sh.cpu().numpy(), shifts)
    np.testing.assert_array_equal(sc.cpu().numpy(), scales)
    np.testing.assert_array_equal(host_u64(words), want_words)
    # int8 operand: value << (8 - bits), element 32w + 8m + t of a chunk at byte 32w + 4t + m
    padded = np.zeros((Q, chunks * 256), dtype=np.int64)
    padded[:, :d] = ints
    e = np.arange(chunks * 256)
    pos = (e // 32) * 32 + ((e % 32) % 8) * 4 + (e % 32) // 8
    want8 = np.zeros_like(padded)
    want8[:, pos] = padded << (8 - bits)
    np.testing.assert_array_equal(i8.cpu().numpy().astype(np.int64), want8)
    # the planes -> int8 pre-pass gives the same bytes
    i8b = torch.zeros_like(i8)
    hip.check(hip.lib.bsi_hip_planes_to_int8(words.data_ptr(), Q, bits, W, i8b.data_ptr(), st()), "p2i8")
    torch.cuda.synchronize()
    assert torch.equal(i8, i8b)


def test_build_huge_magnitudes_take_the_wide_path(hip, oracle):
    """Chunks holding |v * 10^dec| >= 2^31 leave the 32-bit fast path; their neighbours in the same wave do not."""
    x = _inputs(6, 2048, 21)
    x[0, 3] = 3.0e7          # 3e9 after scaling: beyond int32
    x[2, 300] = -5.0e12
    x[5, 2047] = 2.2e7       # 2.2e9: just beyond
    x[4, 1000] = 2.1e7       # 2.1e9: just inside
    ints, shifts, scales = oracle.quantize_fixed(x, 2, 7, True)
    xd = dev(x)
    words = torch.full((6, 7, 32), -1, dtype=torch.int64, device="cuda")
    sh = torch.full(shifts.shape, -1, dtype=torch.int32, device="cuda")
    sc = torch.zeros(scales.shape, dtype=torch.float32, device="cuda")
    i8 = torch.full((6, 2048), 77, dtype=torch.int8, device="cuda")
    hip.check(hip.lib.bsi_hip_build_fixed(xd.data_ptr(), 0, 6, 2048, 2, 7, 1, 0.0, words.data_ptr(), sh.data_ptr(),
                                          sc.data_ptr(), i8.data_ptr(), st()), "build")
    torch.cuda.synchronize()
    np.testing.assert_array_equal(sh.cpu().numpy(), shifts)
    np.testing.assert_array_equal(sc.cpu().numpy(), scales)
    np.testing.assert_array_equal(host_u64(words), oracle.pack(ints, 7))
    e = np.arange(2048)
    pos = (e // 32) * 32 + ((e % 32) % 8) * 4 + (e % 32) // 8
    want8 = np.zeros((6, 2048), dtype=np.int64)
    want8[:, pos] = ints << 1
    np.testing.assert_array_equal(i8.cpu().numpy().astype(np.int64), want8)
    assert shifts.max() >= 30


@pytest.mark.parametrize("Q", [1, 4, 33, 128])
@pytest.mark.parametrize("dt", [torch.float32, torch.float16, torch.bfloat16])
def test_activations_an_int64_cannot_hold(ops, oracle, Q, dt):
    """Infinities, NaNs and magnitudes of 2^63 and more after scaling: the conversion is written out (saturation, NaN ->
    -2^63, as on the reference's hardware) and every route -- the builder, the few-rows kernel with the build inside,
    the one-call layer path -- gives the oracle's planes, scales and outputs for them, bit for bit."""
    rng = np.random.default_rng(Q)
    R, D = 96, 1024
    k = (rng.standard_normal((R, D)) * 0.02).astype(np.float32)
    x = rng.standard_normal((Q, D)).astype(np.float32)
    x[0, 0], x[0, 1], x[-1, 5], x[0, 2], x[0, 3] = np.inf, -np.inf, np.nan, 1e-45, -0.0
    if dt == torch.float32:
        x[0, 300], x[-1, 700], x[0, 600] = 3e38, -1e30, 9.3e16  # 9.3e18 after scaling: just past 2^63
    xt = torch.from_numpy(x).to(dt)
    x = xt.float().numpy()
    qb, kb = oracle.build_queries(x), oracle.build_keys(k)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.5)
    qcap = ops.build_bsi_queries_cuda_batch_packed(xt.cuda(), 2, 0.5)
    np.testing.assert_array_equal(host_u64(qcap.words), qb["words"])
    np.testing.assert_array_equal(qcap.chunk_scales.cpu().numpy(), qb["scales"])
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))
    if Q <= ops.FUSED_LINEAR_MAX_ROWS:
        y = ops.linear_few_rows_cuda(xt.cuda(), kcap, 2)
        np.testing.assert_array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))
    y = ops.linear_cuda(xt.cuda(), kcap, 2)
    np.testing.assert_array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("dec", [0, 1, 2, 3])
@pytest.mark.parametrize("per_wave", [0, 1, 2, 4, 8])
def test_build_rounding_routes_and_items_per_wave(hip, oracle, dec, per_wave):
    """10^dec of 1, 10 and 100 round from the float's mantissa, 1000 in float64; values around the limits of the
    integer route (2^23, ties, denormals, signed zeros) and every items-per-wave variant of the kernel."""
    Q, d = 37, 1024
    rng = np.random.default_rng(dec * 10 + per_wave)
    x = (rng.standard_normal((Q, d)) * 10.0 ** (2 - dec)).astype(np.float32)
    special = np.array([0.125, -0.125, 0.375, 2.5, -2.5, 0.5, -0.5, 1.5, 0.005, -0.005, 0.015, 0.045, 1e-40, -1e-40, 0.0, -0.0,
                        1.17549435e-38, 8388607.5, 8388608.0, -8388607.5, 4194304.25, 4194303.75, 1048576.125, 16777216.0,
                        21474836.0, 21474838.0, 0.49999997, 0.004999999888241291, 0.5000001], dtype=np.float32)
    x[3, :special.size] = special
    x[7, 300:300 + special.size] = -special
    x[11, 512:768] = 0.0
    ints, shifts, scales = oracle.quantize_fixed(x, dec, 7, True)
    xd = dev(x)
    words = torch.full((Q, 7, d // 64), -1, dtype=torch.int64, device="cuda")
    sh = torch.full(shifts.shape, -1, dtype=torch.int32, device="cuda")
    sc = torch.zeros(scales.shape, dtype=torch.float32, device="cuda")
    i8 = torch.full((Q, d), 77, dtype=torch.int8, device="cuda")
    hip.check(hip.lib.bsi_hip_set_option(hip.OPT_BUILD_ITEMS, per_wave), "opt")
    try:
        hip.check(hip.lib.bsi_hip_build_fixed(xd.data_ptr(), 0, Q, d, dec, 7, 1, 0.0, words.data_ptr(), sh.data_ptr(),
                                              sc.data_ptr(), i8.data_ptr(), st()), "build")
        torch.cuda.synchronize()
    finally:
        hip.check(hip.lib.bsi_hip_set_option(hip.OPT_BUILD_ITEMS, 0), "opt")
    np.testing.assert_array_equal(sh.cpu().numpy(), shifts)
    np.testing.assert_array_equal(sc.cpu().numpy(), scales)
    np.testing.assert_array_equal(host_u64(words), oracle.pack(ints, 7))
    e = np.arange(d)
    pos = (e // 32) * 32 + ((e % 32) % 8) * 4 + (e % 32) // 8
    want8 = np.zeros((Q, d), dtype=np.int64)
    want8[:, pos] = ints << 1
    np.testing.assert_array_equal(i8.cpu().numpy().astype(np.int64), want8)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_build_half_inputs(hip, oracle, dtype):
    x = torch.from_numpy(_inputs(12, 1024, 5)).to(dtype)
    ref = x.to(torch.float32).numpy()
    ints, shifts, scales = oracle.quantize_fixed(ref, 2, 7, True)
    xd = x.cuda()
    words = torch.zeros((12, 7, 16), dtype=torch.int64, device="cuda")
    sh = torch.zeros((12, 4), dtype=torch.int32, device="cuda")
    sc = torch.zeros((12, 4), dtype=torch.float32, device="cuda")
    code = 1 if dtype == torch.float16 else 2
    hip.check(hip.lib.bsi_hip_build_fixed(xd.data_ptr(), code, 12, 1024, 2, 7, 1, 0.0, words.data_ptr(), sh.data_ptr(),
                                          sc.data_ptr(), None, st()), "build")
    torch.cuda.synchronize()
    np.testing.assert_array_equal(sh.cpu().numpy(), shifts)
    np.testing.assert_array_equal(host_u64(words), oracle.pack(ints, 7))


def test_build_clip_k(hip, oracle):
    x = _inputs(8, 1024, 3, "outliers")
    for chunk in (True, False):
        ints, shifts, scales = oracle.quantize_fixed(x, 2, 7, chunk, clip_k=6.0)
        assert (shifts != oracle.quantize_fixed(x, 2, 7, chunk)[1]).any()  # clipping changes something
        xd = dev(x)
        words = torch.zeros((8, 7, 16), dtype=torch.int64, device="cuda")
        sh = torch.zeros(shifts.shape, dtype=torch.int32, device="cuda")
        sc = torch.zeros(scales.shape, dtype=torch.float32, device="cuda")
        hip.check(hip.lib.bsi_hip_build_fixed(xd.data_ptr(), 0, 8, 1024, 2, 7, int(chunk), 6.0, words.data_ptr(),
                                              sh.data_ptr(), sc.data_ptr(), None, st()), "build")
        torch.cuda.synchronize()
        np.testing.assert_array_equal(sh.cpu().numpy(), shifts)
        np.testing.assert_array_equal(host_u64(words), oracle.pack(ints, 7))


@pytest.mark.parametrize("Q,d", [(7, 2048), (5, 700), (3, 100)])
def test_staged_builder_entry_points(hip, oracle, Q, d):
    """The separate passes the reference exposes: round -> shift/scale -> shift+clamp -> pack."""
    L = hip.lib
    x = _inputs(Q, d, 11, "outliers")
    xd = dev(x)
    W = (d + 63) // 64
    chunks = (d + 255) // 256
    r = torch.zeros((Q, d), dtype=torch.int64, device="cuda")
    hip.check(L.bsi_hip_quantize_round_to_int64(xd.data_ptr(), 0, Q * d, 100.0, r.data_ptr(), st()), "round")
    torch.cuda.synchronize()
    np.testing.assert_array_equal(r.cpu().numpy(), oracle.round_to_int64(x, 2))
    for chunk in (True, False):
        ints, shifts, scales = oracle.quantize_fixed(x, 2, 7, chunk)
        sh = torch.zeros(shifts.shape, dtype=torch.int32, device="cuda")
        sc = torch.zeros(scales.shape, dtype=torch.float32, device="cuda")
        sh2, sc2 = torch.zeros_like(sh), torch.zeros_like(sc)
        if chunk:
            hip.check(L.bsi_hip_compute_chunk_shift_scale(r.data_ptr(), Q, d, chunks, 7, 0.0, sh.data_ptr(), sc.data_ptr(), st()), "css")
            hip.check(L.bsi_hip_compute_chunk_shift_scale_from_input(xd.data_ptr(), 0, Q, d, chunks, 100.0, 7, 0.0,
                                                                     sh2.data_ptr(), sc2.data_ptr(), st()), "cssi")
        else:
            hip.check(L.bsi_hip_compute_row_shift_scale(r.data_ptr(), Q, d, 7, 0.0, sh.data_ptr(), sc.data_ptr(), st()), "rss")
            hip.check(L.bsi_hip_compute_row_shift_scale_from_input(xd.data_ptr(), 0, Q, d, 100.0, 7, 0.0,
                                                                   sh2.data_ptr(), sc2.data_ptr(), st()), "rssi")
        torch.cuda.synchronize()
        for a, b in ((sh, sc), (sh2, sc2)):
            np.testing.assert_array_equal(a.cpu().numpy(), shifts)
            np.testing.assert_array_equal(b.cpu().numpy(), scales)
        q = r.clone()
        if chunk:
            hip.check(L.bsi_hip_apply_chunk_shift_clamp(q.data_ptr(), Q, d, chunks, sh.data_ptr(), 7, st()), "acsc")
        else:
            hip.check(L.bsi_hip_apply_row_shift_clamp(q.data_ptr(), Q, d, sh.data_ptr(), 7, st()), "arsc")
        torch.cuda.synchronize()
        np.testing.assert_array_equal(q.cpu().numpy(), ints)
        words = torch.zeros((Q, 7, W), dtype=torch.int64, device="cuda")
        hip.check(L.bsi_hip_pack_bits_batch(q.data_ptr(), Q, d, 7, W, words.data_ptr(), st()), "pack")
        words2 = torch.zeros_like(words)
        if chunk:
            hip.check(L.bsi_hip_quantize_shift_pack_chunk_batch(xd.data_ptr(), 0, Q, d, chunks, 7, W, 100.0, 7,
                                                                sh.data_ptr(), words2.data_ptr(), st()), "qspc")
        else:
            hip.check(L.bsi_hip_quantize_shift_pack_row_batch(xd.data_ptr(), 0, Q, d, 7, W, 100.0, 7, sh.data_ptr(),
                                                              words2.data_ptr(), st()), "qspr")
        torch.cuda.synchronize()
        want = oracle.pack(ints, 7)
        np.testing.assert_array_equal(host_u64(words), want)
        np.testing.assert_array_equal(host_u64(words2), want)


# ------------------------------------------------------------------ EWAH


def _ewah_planes(seed, S=14, W=96):
    rng = np.random.default_rng(seed)
    words = rng.integers(0, 2 ** 63, size=(S, W)).astype(np.uint64)
    words[0] = 0
    words[1] = np.uint64(0xFFFFFFFFFFFFFFFF)
    words[2, rng.random(W) < 0.8] = 0
    words[3, rng.random(W) < 0.8] = np.uint64(0xFFFFFFFFFFFFFFFF)
    words[4, 5:50] = 0
    words[4, 50:60] = np.uint64(0xFFFFFFFFFFFFFFFF)
    words[5] = 0
    words[5, 17] = 4096  # 1 bit of 6144: density below the 0.54% cut
    return words


@pytest.mark.parametrize("seed", [0, 1])
def test_ewah_kernels_match_oracle(hip, oracle, seed):
    L = hip.lib
    words = _ewah_planes(seed)
    S, W = words.shape
    wd = dev(words)
    counts = torch.zeros((S,), dtype=torch.int64, device="cuda")
    hip.check(L.bsi_hip_slice_popcount_sum(wd.data_ptr(), S, W, counts.data_ptr(), st()), "pop")
    torch.cuda.synchronize()
    want_counts = np.array([sum(bin(int(v)).count("1") for v in row) for row in words])
    np.testing.assert_array_equal(counts.cpu().numpy(), want_counts)
    for thr in (0.5, 0.0, 1.0):
        flags = torch.zeros((S,), dtype=torch.int32, device="cuda")
        hip.check(L.bsi_hip_compress_flags_from_density(counts.data_ptr(), S, W, thr, flags.data_ptr(), st()), "flags")
        torch.cuda.synchronize()
        want_flags = oracle.compress_flags(words, thr)
        np.testing.assert_array_equal(flags.cpu().numpy(), want_flags)
        stream, off, lens = oracle.ewah_encode(words, want_flags)
        sizes = torch.zeros((S,), dtype=torch.int64, device="cuda")
        hip.check(L.bsi_hip_ewah_size(wd.data_ptr(), S, W, flags.data_ptr(), sizes.data_ptr(), st()), "size")
        torch.cuda.synchronize()
        np.testing.assert_array_equal(sizes.cpu().numpy(), lens)
        offd = dev(off)
        out = torch.zeros((stream.size,), dtype=torch.int64, device="cuda")
        out_len = torch.zeros((S,), dtype=torch.int32, device="cuda")
        hip.check(L.bsi_hip_ewah_emit(wd.data_ptr(), S, W, flags.data_ptr(), offd.data_ptr(), out.data_ptr(),
                                      out_len.data_ptr(), st()), "emit")
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u64(out), stream)
        np.testing.assert_array_equal(out_len.cpu().numpy(), lens)
        back = torch.full((S, W), -1, dtype=torch.int64, device="cuda")
        hip.check(L.bsi_hip_ewah_decompress_batch(out.data_ptr(), offd.data_ptr(), out_len.data_ptr(), S, W,
                                                  back.data_ptr(), st()), "decode")
        one = torch.full((W,), -1, dtype=torch.int64, device="cuda")
        hip.check(L.bsi_hip_ewah_decompress(out.data_ptr() + 8 * int(off[4]), int(lens[4]), W, one.data_ptr(), st()), "decode1")
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u64(back), words)
        np.testing.assert_array_equal(host_u64(one), words[4])


def _codec_round_trip(hip, oracle, words, thr):
    """flags -> size -> emit -> decode on the GPU against the oracle's encoder and decoder."""
    L = hip.lib
    S, W = words.shape
    wd = dev(words)
    flags_np = oracle.compress_flags(words, thr)
    flags = dev(flags_np)
    stream, off, lens = oracle.ewah_encode(words, flags_np)
    sizes = torch.full((S,), -1, dtype=torch.int64, device="cuda")
    hip.check(L.bsi_hip_ewah_size(wd.data_ptr(), S, W, flags.data_ptr(), sizes.data_ptr(), st()), "size")
    offd = dev(off)
    out = torch.full((max(stream.size, 1),), -1, dtype=torch.int64, device="cuda")
    out_len = torch.full((S,), -1, dtype=torch.int32, device="cuda")
    hip.check(L.bsi_hip_ewah_emit(wd.data_ptr(), S, W, flags.data_ptr(), offd.data_ptr(), out.data_ptr(),
                                  out_len.data_ptr(), st()), "emit")
    back = torch.full((S, W), -1, dtype=torch.int64, device="cuda")
    hip.check(L.bsi_hip_ewah_decompress_batch(out.data_ptr(), offd.data_ptr(), out_len.data_ptr(), S, W,
                                              back.data_ptr(), st()), "decode")
    torch.cuda.synchronize()
    np.testing.assert_array_equal(sizes.cpu().numpy(), lens)
    np.testing.assert_array_equal(out_len.cpu().numpy(), lens)
    np.testing.assert_array_equal(host_u64(out)[:stream.size], stream)
    np.testing.assert_array_equal(host_u64(back), words)
    return stream, off, lens


@pytest.mark.parametrize("W", [1, 2, 63, 64, 65, 128, 129, 200, 1000])
def test_ewah_codec_block_edges_and_long_marker_chains(hip, oracle, W):
    """Slices whose runs and literal blocks straddle the 64-word blocks the encoder works in, and streams with far
    more than 64 markers (the decoder's window of stream words is refilled many times)."""
    rng = np.random.default_rng(W)
    ones = np.uint64(0xFFFFFFFFFFFFFFFF)
    rows = []
    lit = rng.integers(1, 2 ** 63, size=W).astype(np.uint64)
    rows.append(lit.copy())                                            # no clean word at all
    rows.append(np.zeros(W, dtype=np.uint64))                          # one run
    rows.append(np.full(W, ones))                                      # one run of ones
    alt = lit.copy(); alt[::2] = 0; rows.append(alt)                   # clean / literal alternating: W / 2 markers
    alt2 = np.zeros(W, dtype=np.uint64); alt2[1::2] = ones; rows.append(alt2)   # zero / one fills alternating: W markers
    blk = lit.copy(); blk[60:70] = 0; blk[70:W // 2 + 70] = ones; rows.append(blk)  # runs across the block edge at 64
    tail = lit.copy(); tail[-1:] = 0; rows.append(tail)                # a run as the last word
    head = lit.copy(); head[0] = ones; rows.append(head)               # a run of one as the first word
    sparse = np.zeros(W, dtype=np.uint64); sparse[rng.integers(0, W, size=max(1, W // 40))] = 1; rows.append(sparse)
    words = np.stack(rows)
    for thr in (1.0, 0.5, 0.0):     # every slice flagged, flagged by density, none flagged
        _codec_round_trip(hip, oracle, words, thr)


def test_ewah_decoder_bounds_match_the_oracle(hip, oracle):
    """Hand-built and damaged streams: a run longer than the slice, literal counts beyond the stream's end, a stream
    cut short, trailing words after the slice is full, an empty stream -- decoded as the oracle's restatement of the
    reference decoder does (output clipped at W, input at its length, the rest zero)."""
    L = hip.lib
    W = 70

    def marker(bit, run, lit):
        return np.uint64(bit | (run << 1) | (lit << 33))

    lits = np.arange(1, 200, dtype=np.uint64) * np.uint64(0x0101010101010101)
    streams = [
        np.array([marker(1, 500, 0)], dtype=np.uint64),                                   # run beyond W
        np.concatenate([[marker(0, 3, 100)], lits[:20]]),                                 # literal count beyond the input
        np.concatenate([[marker(0, 0, 10)], lits[:10], [marker(1, 5, 2)], lits[10:11]]),  # second block cut short
        np.concatenate([[marker(0, 60, 10)], lits[:10], [marker(1, 9, 9)], lits[10:19]]),  # words left after W
        np.zeros(0, dtype=np.uint64),                                                     # nothing at all
        np.concatenate([[marker(0, 0, 0)], [marker(1, 2, 1)], lits[:1]]),                 # an empty marker first
        np.concatenate([np.array([marker(0, 1, 0), marker(1, 1, 0)] * 35, dtype=np.uint64)]),  # 70 markers, no literal
    ]
    for strm in streams:
        want = oracle.ewah_decompress(strm, W)
        buf = dev(strm if strm.size else np.zeros(1, dtype=np.uint64))
        one = torch.full((W,), -1, dtype=torch.int64, device="cuda")
        hip.check(L.bsi_hip_ewah_decompress(buf.data_ptr(), int(strm.size), W, one.data_ptr(), st()), "decode1")
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u64(one), want)


def test_hybrid_query_builder(ops, oracle):
    x = np.maximum(_inputs(1, 8192, 4), 0)[0]  # ReLU: sign plane all zero
    cap, mem, S, W = ops.build_bsi_query_cuda_hybrid(torch.from_numpy(x).cuda(), 2, 0.5)
    cap2, mem2, S2, W2 = ops.build_bsi_query_cuda(torch.from_numpy(x).cuda(), 2, 0.5)
    torch.cuda.synchronize()
    assert (S, W) == (7, 128) == (S2, W2)
    assert torch.equal(cap.dev_words, cap2.dev_words)  # decode(encode(x)) == x
    ints, shifts, scales = oracle.quantize_fixed(x[None], 2, 7, False)
    planes = oracle.pack(ints, 7)[0]
    np.testing.assert_array_equal(host_u64(cap.dev_words), planes)
    stream, off, lens = oracle.ewah_encode(planes, oracle.compress_flags(planes, 0.5))
    np.testing.assert_array_equal(host_u64(cap.comp_words), stream)
    np.testing.assert_array_equal(cap.comp_len.cpu().numpy(), lens)
    assert lens[6] == 1 and mem == (stream.size + 7 * 128) * 8 and mem2 == 7 * 128 * 8
    assert not cap2.twos_complement and float(cap.slice_weights[0]) == float(scales[0])


# ------------------------------------------------------------------ dot through the raw C ABI


def _oracle_case(oracle, Q, R, d, seed, qkind="randn", ksigma=0.02, bits_q=7, bits_k=6):
    x = _inputs(Q, d, seed, qkind)
    rng = np.random.default_rng(seed + 1000)
    k = (rng.standard_normal((R, d)) * ksigma).astype(np.float32)
    if R > 3:
        k[3] *= 50  # one row with a large key shift
    qb = oracle.build_queries(x, 2, bits_q)
    kb = oracle.build_keys(k, 2, bits_k)
    ints, out = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    return x, k, qb, kb, ints, out


# forms of the `tiled` argument that select the cached int8 key image, and the tile each one forces (0: automatic)
_I8_TILES = {"int8": 0, "int8-128": 128, "int8-1284": 1284, "int8-12864": 12864, "int8-64": 64, "int8-6432": 6432}


def _run_dot(hip, qb, kb, Q, R, W, Sa, Sb, core, tiled, with_ints8, want_ints=True, R_total=None):
    """One bsi_hip_dot call.  With the int8 key image the call is made twice, on the row-major image and on the
    image tiled by 64 rows and half-chunks, and both must give the same bits."""
    if tiled in _I8_TILES:
        ints_a, out_a = _run_dot_once(hip, qb, kb, Q, R, W, Sa, Sb, core, tiled, with_ints8, want_ints, R_total, False)
        ints_b, out_b = _run_dot_once(hip, qb, kb, Q, R, W, Sa, Sb, core, tiled, with_ints8, want_ints, R_total, True)
        assert np.array_equal(out_a, out_b, equal_nan=True)
        assert ints_a is None or np.array_equal(ints_a, ints_b)
        return ints_b, out_b
    return _run_dot_once(hip, qb, kb, Q, R, W, Sa, Sb, core, tiled, with_ints8, want_ints, R_total, False)


def _run_dot_once(hip, qb, kb, Q, R, W, Sa, Sb, core, tiled, with_ints8, want_ints, R_total, image_tiled):
    L = hip.lib
    chunks = (W + 3) // 4
    A = dev(qb["words"])
    scales = dev(qb["scales"])
    stride = chunks if qb["chunk_scale"] else 1
    B = dev(kb["words"])
    layout = 0
    if tiled in _I8_TILES:   # the cached int8 image of the key integers; tile forced or automatic
        hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, _I8_TILES[tiled]), "set_option")
        if image_tiled:
            Bi = torch.full((int(L.bsi_hip_int8_tiled_bytes(R, W)),), 77, dtype=torch.int8, device="cuda")
            hip.check(L.bsi_hip_planes_to_int8_tiled(B.data_ptr(), R, Sb, W, Bi.data_ptr(), st()), "key image")
            B, layout = Bi, 3
        else:
            Bi = torch.full((R, chunks * 256), 77, dtype=torch.int8, device="cuda")
            hip.check(L.bsi_hip_planes_to_int8(B.data_ptr(), R, Sb, W, Bi.data_ptr(), st()), "key image")
            B, layout = Bi, 2
    elif tiled:
        Bt = torch.full((((R + 15) // 16) * chunks * Sb * 64,), -1, dtype=torch.int64, device="cuda")
        hip.check(L.bsi_hip_tile_key_planes(B.data_ptr(), R, Sb, W, Bt.data_ptr(), st()), "tile")
        B, layout = Bt, 1
    Bw = dev(kb["slice_weights"])
    a8 = None
    if with_ints8:
        a8 = torch.zeros((Q, chunks * 256), dtype=torch.int8, device="cuda")
        hip.check(L.bsi_hip_planes_to_int8(A.data_ptr(), Q, Sa, W, a8.data_ptr(), st()), "p2i8")
    R_total = R if R_total is None else R_total
    out = torch.full((Q, R_total), float("nan"), dtype=torch.float32, device="cuda")
    ints = torch.full((Q, R, chunks), -7, dtype=torch.int32, device="cuda") if want_ints else None
    ws_bytes = int(L.bsi_hip_dot_workspace_bytes(Q, W, core))
    ws = torch.zeros((max(ws_bytes, 16),), dtype=torch.uint8, device="cuda")
    hip.check(L.bsi_hip_dot(A.data_ptr(), a8.data_ptr() if a8 is not None else None, scales.data_ptr(), stride, Sa, W,
                            B.data_ptr(), layout, Bw.data_ptr(), Sb, R, Q, float(np.float32(1e-4)), R_total,
                            out.data_ptr(), ints.data_ptr() if ints is not None else None, core, ws.data_ptr(),
                            ws_bytes, st()), "dot")
    torch.cuda.synchronize()
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, 0), "set_option")
    return (ints.cpu().numpy() if ints is not None else None), out.cpu().numpy()


DOT_SHAPES = [
    (64, 256, 2048, "randn"),     # the correctness-scale configuration
    (37, 75, 2048, "outliers"),   # ragged Q and R
    (130, 129, 512, "relu"),      # tile edges on both sides, ReLU queries
    (5, 3, 256, "ties"),          # a single chunk
    (16, 40, 700, "randn"),       # W64 = 11: row scale, partial last chunk
    (1, 200, 4096, "randn"),      # a single query
    (17, 50, 1024, "randn"),      # two query tiles of the few-rows kernel, ragged in both
    (32, 33, 8704, "relu"),       # 34 chunks: more than one pass of the few-rows kernel with two query tiles
    (3, 20, 16640, "randn"),      # 65 chunks: more than one pass with one query tile
    (3, 16400, 256, "randn"),     # many key tiles: two per workgroup in the few-rows kernel, last tile ragged
    (20, 16390, 512, "relu"),     # the same with two query tiles
]


@pytest.mark.parametrize("Q,R,d,kind", DOT_SHAPES)
@pytest.mark.parametrize("core,tiled,ints8", [(1, False, False), (1, True, False), (2, False, True), (2, True, False),
                                              (0, True, True), (2, "int8-128", True), (0, "int8-64", False),
                                              (2, "int8-12864", True), (0, "int8-12864", False),
                                              (2, "int8-6432", True), (0, "int8-6432", False),
                                              (2, "int8-1284", True), (0, "int8-1284", False)])
def test_dot_bit_exact(hip, oracle, Q, R, d, kind, core, tiled, ints8):
    x, k, qb, kb, want_ints, want_out = _oracle_case(oracle, Q, R, d, seed=Q + R + d, qkind=kind)
    W = (d + 63) // 64
    ints, out = _run_dot(hip, qb, kb, Q, R, W, 7, 6, core, tiled, ints8)
    np.testing.assert_array_equal(ints, want_ints)                     # integer accumulators: bit-exact
    np.testing.assert_allclose(out, want_out, rtol=FP32_RTOL, atol=0)  # the stated fp32 bar
    np.testing.assert_array_equal(out, want_out)                       # and in fact identical
    # independent of the popcount form: the accumulators are the integer dot of the quantised values
    c0 = qb["ints"][:, :256] @ kb["ints"][:, :256].T
    np.testing.assert_array_equal(ints[:, :, 0], c0)
    if core != 1:
        # the production launch (no accumulator dump) is a different kernel instance: same floats
        _, out2 = _run_dot(hip, qb, kb, Q, R, W, 7, 6, core, tiled, ints8, want_ints=False)
        np.testing.assert_array_equal(out2, want_out)


@pytest.mark.parametrize("R,d,kind,force", [(75, 2048, "relu", False), (200, 4096, "randn", True), (40, 700, "relu", True),
                                            (20, 16640, "relu", False), (33, 256, "ties", True)])
def test_dot_ewah_query_inline(hip, oracle, R, d, kind, force):
    """One query handed over as EWAH streams, decoded inside the dot: identical to the dot on verbatim planes."""
    x, k, qb, kb, want_ints, want_out = _oracle_case(oracle, 1, R, d, seed=R + d, qkind=kind)
    L = hip.lib
    W = (d + 63) // 64
    chunks = (W + 3) // 4
    planes = qb["words"][0]
    flags = np.ones(7, dtype=np.int32) if force else oracle.compress_flags(planes, 0.5)
    stream, off, lens = oracle.ewah_encode(planes, flags)
    if kind == "relu" and not force:
        assert lens[6] == 1  # the all-zero sign plane is one run marker
    comp, offd, lend = dev(stream), dev(off.astype(np.int64)), dev(lens.astype(np.int32))
    scales = dev(qb["scales"])
    stride = chunks if qb["chunk_scale"] else 1
    B = dev(kb["words"])
    Bt = torch.full((((R + 15) // 16) * chunks * 6 * 64,), -1, dtype=torch.int64, device="cuda")
    hip.check(L.bsi_hip_tile_key_planes(B.data_ptr(), R, 6, W, Bt.data_ptr(), st()), "tile")
    Bw = dev(kb["slice_weights"])
    for with_ints in (True, False):
        out = torch.full((R,), float("nan"), dtype=torch.float32, device="cuda")
        ints = torch.full((R, chunks), -7, dtype=torch.int32, device="cuda") if with_ints else None
        hip.check(L.bsi_hip_dot_ewah_query(comp.data_ptr(), offd.data_ptr(), lend.data_ptr(), 7, W, scales.data_ptr(),
                                           stride, Bt.data_ptr(), Bw.data_ptr(), 6, R, float(np.float32(1e-4)),
                                           out.data_ptr(), ints.data_ptr() if with_ints else None, st()), "ewah dot")
        torch.cuda.synchronize()
        if with_ints:
            np.testing.assert_array_equal(ints.cpu().numpy(), want_ints[0])
        np.testing.assert_array_equal(out.cpu().numpy(), want_out[0])
    rc = L.bsi_hip_dot_ewah_query(comp.data_ptr(), offd.data_ptr(), lend.data_ptr(), 7, W, scales.data_ptr(), stride,
                                  Bt.data_ptr(), Bw.data_ptr(), 5, R, 1.0, out.data_ptr(), None, st())
    assert rc == 3  # only 6-plane keys


def test_hybrid_query_dot_decodes_inline(ops, oracle, monkeypatch):
    x = np.maximum(_inputs(1, 4096, 11), 0)[0]
    rng = np.random.default_rng(5)
    k = (rng.standard_normal((300, 4096)) * 0.02).astype(np.float32)
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.5)
    cap, *_ = ops.build_bsi_query_cuda_hybrid(torch.from_numpy(x).cuda(), 2, 0.5)
    out, *_ = ops.batch_dot_product_multiquery_cuda_caps([cap], kcap)       # streams decoded in the kernel
    monkeypatch.setenv("BSI_EWAH_INLINE", "0")
    ops._reset_flag_cache()
    ref, *_ = ops.batch_dot_product_multiquery_cuda_caps([cap], kcap)       # verbatim planes
    assert out.shape == (1, 300) and torch.equal(out, ref)
    qi, _, qscale = oracle.quantize_fixed(x[None], 2, 7, False)   # a single query vector carries one row scale
    kb = oracle.build_keys(k)
    _, want = oracle.dot_fixed(oracle.pack(qi, 7), qscale, kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    np.testing.assert_array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("Sa,Sb", [(8, 8), (5, 4), (2, 2), (7, 5), (3, 7)])
@pytest.mark.parametrize("core,tiled", [(1, False), (1, True), (2, True), (2, "int8-128"), (2, "int8-1284"), (2, "int8-12864"), (2, "int8-64"), (2, "int8-6432")])
def test_dot_other_bit_widths(hip, oracle, Sa, Sb, core, tiled):
    Q, R, d = 19, 35, 1024
    x, k, qb, kb, want_ints, want_out = _oracle_case(oracle, Q, R, d, seed=Sa * 10 + Sb, ksigma=0.05, bits_q=Sa, bits_k=Sb)
    ints, out = _run_dot(hip, qb, kb, Q, R, 16, Sa, Sb, core, tiled=tiled, with_ints8=False)
    np.testing.assert_array_equal(ints, want_ints)
    np.testing.assert_array_equal(out, want_out)


@pytest.mark.parametrize("Sa,Sb", [(7, 1), (1, 6), (1, 1), (9, 1), (2, 1), (1, 12)])
@pytest.mark.parametrize("core", [0, 1])
def test_dot_single_slice_operands(hip, oracle, Sa, Sb, core):
    """One-bit two's-complement operands hold 0 and -1: their only slice is the sign slice, and the keys' slice-0
    weight, which the dots use as the row scale, is then negative.  The sign of the products is in the plane signs
    alone: outputs and integer accumulators are the oracle's.  (The matrix-core route takes 2 to 8 bits and says so.)"""
    Q, R, d = 21, 37, 768
    x, k, qb, kb, want_ints, want_out = _oracle_case(oracle, Q, R, d, seed=Sa * 20 + Sb, ksigma=0.05, bits_q=Sa, bits_k=Sb)
    if Sb == 1:
        assert (kb["slice_weights"] < 0).all() and set(np.unique(kb["ints"])) <= {0, -1}
    ints, out = _run_dot(hip, qb, kb, Q, R, 12, Sa, Sb, core, tiled=False, with_ints8=False)
    np.testing.assert_array_equal(ints, want_ints)
    np.testing.assert_array_equal(out, want_out)
    assert np.any(want_out != 0)
    L = hip.lib
    t = torch.zeros(64, device="cuda")
    rc = L.bsi_hip_dot(t.data_ptr(), None, t.data_ptr(), 1, Sa, 1, t.data_ptr(), 0, t.data_ptr(), Sb, 1, 1, 1.0, 1,
                       t.data_ptr(), None, 2, t.data_ptr(), 256, st())
    if min(Sa, Sb) == 1 or max(Sa, Sb) > 8:
        assert rc == 3 and b"MFMA core needs" in L.bsi_hip_last_error()


def test_dot_wide_planes_valu_only(hip, oracle):
    Q, R, d = 6, 10, 512
    x, k, qb, kb, want_ints, want_out = _oracle_case(oracle, Q, R, d, seed=99, ksigma=0.5, bits_q=12, bits_k=10)
    for tiled in (False, True):
        ints, out = _run_dot(hip, qb, kb, Q, R, 8, 12, 10, 0, tiled=tiled, with_ints8=False)  # auto -> VALU
        np.testing.assert_array_equal(ints, want_ints)
        np.testing.assert_array_equal(out, want_out)
    L = hip.lib
    t = torch.zeros(8, device="cuda")
    rc = L.bsi_hip_dot(t.data_ptr(), None, t.data_ptr(), 2, 12, 8, t.data_ptr(), 0, t.data_ptr(), 10, 1, 1, 1.0, 1,
                       t.data_ptr(), None, 2, None, 0, st())
    assert rc == 3 and b"MFMA core needs" in L.bsi_hip_last_error()


def test_dot_extreme_values(hip, oracle):
    # every product at its largest magnitude: I = 2^19 per chunk, both signs
    Q, R, d = 4, 6, 1024
    a = np.full((Q, d), -64, dtype=np.int64)
    a[1] = 63
    b = np.full((R, d), -32, dtype=np.int64)
    b[2] = 31
    qb = dict(words=oracle.pack(a, 7), scales=np.full((Q, 4), 8, np.float32), chunk_scale=True)
    kb = dict(words=oracle.pack(b, 6), slice_weights=(oracle.slice_weights(6)[None] * np.ones((R, 1), np.float32)))
    want_ints, want_out = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], np.ones(R, np.float32), np.float32(1e-4))
    assert want_ints.max() == 1 << 19
    for core in (1, 2):
        ints, out = _run_dot(hip, qb, kb, Q, R, 16, 7, 6, core, tiled=True, with_ints8=False)
        np.testing.assert_array_equal(ints, want_ints)
        np.testing.assert_array_equal(out, want_out)


def test_dot_fp32_rounding_order(hip, oracle):
    # 40 chunks of same-sign products with mixed scales: the fp32 accumulator rounds, so only the
    # reference's chunk order reproduces the bits
    rng = np.random.default_rng(11)
    Q, R, d = 8, 24, 256 * 40
    a = rng.integers(40, 64, size=(Q, d)).astype(np.int64)
    b = rng.integers(20, 32, size=(R, d)).astype(np.int64)
    a[1] = -a[1]
    qb = dict(words=oracle.pack(a, 7), scales=(2.0 ** rng.integers(0, 8, size=(Q, 40))).astype(np.float32), chunk_scale=True)
    bscale = (2.0 ** rng.integers(0, 5, size=R)).astype(np.float32)
    kb = dict(words=oracle.pack(b, 6), slice_weights=(oracle.slice_weights(6)[None] * bscale[:, None]).astype(np.float32))
    want_ints, want_out = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], bscale, np.float32(1e-4))
    for core in (1, 2):
        ints, out = _run_dot(hip, qb, kb, Q, R, 160, 7, 6, core, tiled=False, with_ints8=True)
        np.testing.assert_array_equal(ints, want_ints)
        np.testing.assert_array_equal(out, want_out)


def test_dot_row_stride_and_untouched_columns(hip, oracle):
    Q, R, d = 10, 20, 512
    x, k, qb, kb, want_ints, want_out = _oracle_case(oracle, Q, R, d, seed=5)
    for core in (1, 2):
        _, out = _run_dot(hip, qb, kb, Q, R, 8, 7, 6, core, tiled=True, with_ints8=False, want_ints=False, R_total=27)
        np.testing.assert_array_equal(out[:, :R], want_out)
        assert np.isnan(out[:, R:]).all()  # columns past R are not written


def test_dot_row_stride_int8_image_and_few_rows(hip, oracle):
    x, k, qb, kb, want_ints, want_out = _oracle_case(oracle, 70, 150, 1024, seed=8)
    for tiled in ("int8-128", "int8-1284", "int8-12864", "int8-64", "int8-6432"):
        _, out = _run_dot(hip, qb, kb, 70, 150, 16, 7, 6, 2, tiled=tiled, with_ints8=True, want_ints=False, R_total=163)
        np.testing.assert_array_equal(out[:, :150], want_out)
        assert np.isnan(out[:, 150:]).all()
    x, k, qb, kb, want_ints, want_out = _oracle_case(oracle, 9, 150, 1024, seed=9)
    _, out = _run_dot(hip, qb, kb, 9, 150, 16, 7, 6, 2, tiled=True, with_ints8=True, want_ints=False, R_total=163)
    np.testing.assert_array_equal(out[:, :150], want_out)
    assert np.isnan(out[:, 150:]).all()


@pytest.mark.parametrize("tile", ["int8-128", "int8-1284", "int8-12864", "int8-64", "int8-6432"])
@pytest.mark.parametrize("d", [256, 512, 768, 1280, 1792, 2304, 4352])
def test_dot_int8_image_short_and_odd_chunk_counts(hip, oracle, d, tile):
    """1, 2, 3, 5, 7, 9 and 17 chunks through every tile of the int8-image kernel: the loader's prologue (three stages
    ahead of a loop that may have fewer) and its tail (no loads behind the last stage) meet the MFMA waves' barriers
    one for one; outputs and per-chunk integers bit-identical to the oracle, with and without bias."""
    Q, R, W = 70, 150, d // 64
    chunks = d // 256
    x, k, qb, kb, want_ints, want_out = _oracle_case(oracle, Q, R, d, seed=d)
    bias = np.random.default_rng(d).standard_normal(R).astype(np.float32)
    L = hip.lib
    A, scales, Bc, Bw = dev(qb["words"]), dev(qb["scales"]), dev(kb["words"]), dev(kb["slice_weights"])
    a8 = torch.zeros((Q, chunks * 256), dtype=torch.int8, device="cuda")
    hip.check(L.bsi_hip_planes_to_int8(A.data_ptr(), Q, 7, W, a8.data_ptr(), st()), "p2i8")
    B = torch.zeros((R, chunks * 256), dtype=torch.int8, device="cuda")
    hip.check(L.bsi_hip_planes_to_int8(Bc.data_ptr(), R, 6, W, B.data_ptr(), st()), "image")
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, _I8_TILES[tile]), "opt")
    try:
        out = torch.full((Q, R), float("nan"), dtype=torch.float32, device="cuda")
        ints = torch.full((Q, R, chunks), -7, dtype=torch.int32, device="cuda")
        hip.check(L.bsi_hip_dot(A.data_ptr(), a8.data_ptr(), scales.data_ptr(), chunks, 7, W, B.data_ptr(), 2, Bw.data_ptr(),
                                6, R, Q, float(np.float32(1e-4)), R, out.data_ptr(), ints.data_ptr(), 2, None, 0, st()), "dot")
        outb = torch.full((Q, R), float("nan"), dtype=torch.float32, device="cuda")
        bias_d = dev(bias)  # named, so that it lives until the kernel has run
        hip.check(L.bsi_hip_dot_bias(A.data_ptr(), a8.data_ptr(), scales.data_ptr(), chunks, 7, W, B.data_ptr(), 2,
                                     Bw.data_ptr(), 6, R, Q, float(np.float32(1e-4)), R, bias_d.data_ptr(),
                                     outb.data_ptr(), 2, None, 0, st()), "dot_bias")
        torch.cuda.synchronize()
    finally:
        hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, 0), "opt")
    np.testing.assert_array_equal(ints.cpu().numpy(), want_ints)
    np.testing.assert_array_equal(out.cpu().numpy(), want_out)
    np.testing.assert_array_equal(outb.cpu().numpy(), want_out + bias[None, :])


@pytest.mark.parametrize("tile", ["int8-128", "int8-1284", "int8-12864", "int8-64", "int8-6432"])
@pytest.mark.parametrize("stores", [0, 1, 2])
def test_dot_whole_tiles_stored_in_lines(hip, oracle, tile, stores):
    """Output tiles that lie wholly inside an aligned output are stored in whole 128-byte lines after a lane exchange,
    with plain or nontemporal stores (BSI_OPT_OUTPUT_STORES; 0 = plain from the layer entry point bsi_hip_dot_bias,
    nontemporal from bsi_hip_dot).  The last key tile and the last query tile are ragged and take the element path;
    every combination must give the oracle's bits, through both entry points."""
    Q, R, d, W = 200, 416, 1024, 16  # 416 = 13 x 32: the lines are aligned, the last tile of 64 or 128 keys is not whole
    x, k, qb, kb, want_ints, want_out = _oracle_case(oracle, Q, R, d, seed=77)
    bias = np.random.default_rng(2).standard_normal(R).astype(np.float32)
    L = hip.lib
    A, scales, Bc, Bw, bd = dev(qb["words"]), dev(qb["scales"]), dev(kb["words"]), dev(kb["slice_weights"]), dev(bias)
    a8 = torch.zeros((Q, 4 * 256), dtype=torch.int8, device="cuda")
    hip.check(L.bsi_hip_planes_to_int8(A.data_ptr(), Q, 7, W, a8.data_ptr(), st()), "p2i8")
    B = torch.zeros((R, 4 * 256), dtype=torch.int8, device="cuda")
    hip.check(L.bsi_hip_planes_to_int8(Bc.data_ptr(), R, 6, W, B.data_ptr(), st()), "image")
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, _I8_TILES[tile]), "opt")
    hip.check(L.bsi_hip_set_option(hip.OPT_OUTPUT_STORES, stores), "opt")
    try:
        out = torch.full((Q, R), float("nan"), dtype=torch.float32, device="cuda")
        hip.check(L.bsi_hip_dot(A.data_ptr(), a8.data_ptr(), scales.data_ptr(), 4, 7, W, B.data_ptr(), 2, Bw.data_ptr(), 6,
                                R, Q, float(np.float32(1e-4)), R, out.data_ptr(), None, 2, None, 0, st()), "dot")
        outb = torch.full((Q, R), float("nan"), dtype=torch.float32, device="cuda")
        hip.check(L.bsi_hip_dot_bias(A.data_ptr(), a8.data_ptr(), scales.data_ptr(), 4, 7, W, B.data_ptr(), 2,
                                     Bw.data_ptr(), 6, R, Q, float(np.float32(1e-4)), R, bd.data_ptr(), outb.data_ptr(),
                                     2, None, 0, st()), "dot_bias")
        # an output whose base is not on a 128-byte line (64 bytes off), and one 4 bytes off: the element paths
        off = []
        for shift in (16, 1):
            flat = torch.full((Q * R + 32,), float("nan"), dtype=torch.float32, device="cuda")
            hip.check(L.bsi_hip_dot(A.data_ptr(), a8.data_ptr(), scales.data_ptr(), 4, 7, W, B.data_ptr(), 2, Bw.data_ptr(),
                                    6, R, Q, float(np.float32(1e-4)), R, flat.data_ptr() + 4 * shift, None, 2, None, 0, st()),
                      "dot")
            off.append((shift, flat))
        torch.cuda.synchronize()
    finally:
        hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, 0), "opt")
        hip.check(L.bsi_hip_set_option(hip.OPT_OUTPUT_STORES, 0), "opt")
    np.testing.assert_array_equal(out.cpu().numpy(), want_out)
    np.testing.assert_array_equal(outb.cpu().numpy(), want_out + bias[None, :])
    for shift, flat in off:
        got = flat.cpu().numpy()
        np.testing.assert_array_equal(got[shift:shift + Q * R].reshape(Q, R), want_out)
        assert np.isnan(got[:shift]).all() and np.isnan(got[shift + Q * R:]).all()


@pytest.mark.parametrize("Q,tiled", [(70, "int8-128"), (70, "int8-1284"), (70, "int8-12864"), (70, "int8-64"), (70, "int8-6432"), (9, True), (70, True), (70, False)])
def test_dot_bias_entry_point(hip, oracle, Q, tiled):
    """bsi_hip_dot_bias == bsi_hip_dot followed by a float addition of the bias row, bit for bit, whether the
    kernel adds it in its epilogue (int8 image, few rows) or the library appends an addition kernel."""
    R, d, W = 150, 1024, 16
    x, k, qb, kb, want_ints, want_out = _oracle_case(oracle, Q, R, d, seed=Q)
    rng = np.random.default_rng(1)
    bias = rng.standard_normal(R).astype(np.float32)
    L = hip.lib
    A, scales, Bc, Bw = dev(qb["words"]), dev(qb["scales"]), dev(kb["words"]), dev(kb["slice_weights"])
    a8 = torch.zeros((Q, 4 * 256), dtype=torch.int8, device="cuda")
    hip.check(L.bsi_hip_planes_to_int8(A.data_ptr(), Q, 7, W, a8.data_ptr(), st()), "p2i8")
    if tiled in _I8_TILES:
        hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, _I8_TILES[tiled]), "opt")
        B = torch.zeros((R, 4 * 256), dtype=torch.int8, device="cuda")
        hip.check(L.bsi_hip_planes_to_int8(Bc.data_ptr(), R, 6, W, B.data_ptr(), st()), "image")
        layout = 2
    elif tiled:
        B = torch.zeros((((R + 15) // 16) * 4 * 6 * 64,), dtype=torch.int64, device="cuda")
        hip.check(L.bsi_hip_tile_key_planes(Bc.data_ptr(), R, 6, W, B.data_ptr(), st()), "tile")
        layout = 1
    else:
        B, layout = Bc, 0
    bd = dev(bias)
    out = torch.full((Q, R + 5), float("nan"), dtype=torch.float32, device="cuda")
    hip.check(L.bsi_hip_dot_bias(A.data_ptr(), a8.data_ptr(), scales.data_ptr(), 4, 7, W, B.data_ptr(), layout,
                                 Bw.data_ptr(), 6, R, Q, float(np.float32(1e-4)), R + 5, bd.data_ptr(), out.data_ptr(),
                                 2, None, 0, st()), "dot_bias")
    torch.cuda.synchronize()
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, 0), "opt")
    got = out.cpu().numpy()
    np.testing.assert_array_equal(got[:, :R], want_out + bias[None, :])
    assert np.isnan(got[:, R:]).all()


def test_build_and_dot_replay_from_a_hip_graph(ops):
    """Query build + dot launched on a side stream are captured once and replayed; every replay, with
    eager work and synchronisations between them, gives the eager result for the input then in place."""
    torch.manual_seed(3)
    K = torch.randn(300, 1024) * 0.02
    kcap, *_ = ops.build_bsi_keys_cuda(K, 2, 0.5)
    xs = [torch.randn(40, 1024, device="cuda") for _ in range(3)]
    xs_few = [torch.randn(5, 1024, device="cuda") for _ in range(3)]
    for inputs in (xs, xs_few):   # the int8-image kernel, then the few-rows kernel
        eager = []
        for xi in inputs:
            qc = ops.build_bsi_queries_cuda_batch_packed(xi, 2, 0.5)
            eager.append(ops.batch_dot_product_multiquery_cuda_batch_caps(qc, kcap)[0].clone())
        static_x = inputs[0].clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            qc = ops.build_bsi_queries_cuda_batch_packed(static_x, 2, 0.5)
            ops.batch_dot_product_multiquery_cuda_batch_caps(qc, kcap)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            qc = ops.build_bsi_queries_cuda_batch_packed(static_x, 2, 0.5)
            static_out = ops.batch_dot_product_multiquery_cuda_batch_caps(qc, kcap)[0]
        for rep in range(2):
            for xi, want in zip(inputs, eager):
                static_x.copy_(xi)
                g.replay()
                torch.cuda.synchronize()
                assert torch.equal(static_out, want)
                other = ops.build_bsi_queries_cuda_batch_packed(inputs[(rep + 1) % 3], 2, 0.5)   # eager work in between
                ops.batch_dot_product_multiquery_cuda_batch_caps(other, kcap)
                torch.cuda.synchronize()


# ------------------------------------------------------------------ through the bsi_ops mirror


@pytest.mark.parametrize("bq,bk", [(9, 6), (7, 10), (12, 10), (16, 16), (2, 2), (8, 8), (4, 9)])
@pytest.mark.parametrize("Q,R,D", [(1, 50, 512), (20, 100, 1024), (140, 130, 768), (3, 40, 700)])
def test_ops_other_fixed_bit_widths(ops, oracle, monkeypatch, bq, bk, Q, R, D):
    """BSI_FIXED_BITS_QUERIES / BSI_FIXED_BITS_KEYS other than 7 / 6, wider than the matrix cores take included: the
    keys are kept tiled all the same, and the popcount kernel for any width reads them there (it used to refuse every
    layout but the canonical one, so such a dot failed from 33 rows up and for rows without chunk scales)."""
    monkeypatch.setenv("BSI_FIXED_BITS_QUERIES", str(bq))
    monkeypatch.setenv("BSI_FIXED_BITS_KEYS", str(bk))
    ops._reset_flag_cache()
    rng = np.random.default_rng(bq * 100 + bk + Q)
    x = rng.standard_normal((Q, D)).astype(np.float32)
    k = (rng.standard_normal((R, D)) * 0.05).astype(np.float32)
    qb, kb = oracle.build_queries(x, 2, bq), oracle.build_keys(k, 2, bk)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.5)
    qcap = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(x).cuda(), 2, 0.5)
    assert qcap.Sa == bq and kcap.Sb == bk
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("bq,bk", [(17, 17), (20, 33), (32, 32), (63, 63)])
@pytest.mark.parametrize("Q,R,D", [(1, 50, 512), (40, 100, 1024), (3, 40, 700)])
def test_ops_fixed_bit_widths_up_to_63(ops, oracle, monkeypatch, bq, bk, Q, R, D):
    """The reference takes fixed-bit flags up to 63 (bsi_vector_cuda.cpp:256-262).  With 17 bits and more nothing of
    these inputs is shifted away, so every chunk's integer is the integer dot of the values rounded at two decimals
    (numpy int64) and the output is the fp32 chain over those integers, replayed here in float64 with one rounding
    per step: bit for bit."""
    monkeypatch.setenv("BSI_FIXED_BITS_QUERIES", str(bq))
    monkeypatch.setenv("BSI_FIXED_BITS_KEYS", str(bk))
    ops._reset_flag_cache()
    rng = np.random.default_rng(bq + bk + Q)
    x = rng.standard_normal((Q, D)).astype(np.float32)
    k = (rng.standard_normal((R, D)) * 0.05).astype(np.float32)
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.5)
    qcap = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(x).cuda(), 2, 0.5)
    assert qcap.Sa == bq and kcap.Sb == bk
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    xi, ki = oracle.round_to_int64(x, 2), oracle.round_to_int64(k, 2)
    assert np.abs(xi).max() < 2 ** 16 and np.abs(ki).max() < 2 ** 16
    acc = np.zeros((Q, R), dtype=np.float32)
    for c0 in range(0, D, 256):
        I = xi[:, c0:c0 + 256] @ ki[:, c0:c0 + 256].T
        assert np.abs(I).max() < 2 ** 24  # exact as float32
        acc = (I.astype(np.float64) + acc.astype(np.float64)).astype(np.float32)  # fmaf(float(I), 1, acc)
    want = acc * oracle.scale_inv(2, 2)
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_reference_known_answers_gpu(ops, monkeypatch):
    kat = json.load(open(GOLDEN))
    for case in kat["vector_dot"] + kat["batch_dot"]:
        monkeypatch.setenv("BSI_FIXED_BITS_KEYS", str(case["key_bits"]))
        ops._reset_flag_cache()
        q = torch.tensor(case["q"] if "K" in case else [case["q"]], dtype=torch.float32)
        K = torch.tensor(case["K"] if "K" in case else [case["k"]], dtype=torch.float32)
        dec = case["decimal_places"]
        kcap, nbytes, nk, d, W = ops.build_bsi_keys_cuda(K, dec, 0.2)
        assert (nk, d, W) == (K.shape[0], K.shape[1], 1) and nbytes == nk * case["key_bits"] * 8
        qcap = ops.build_bsi_queries_cuda_batch_packed(q.cuda(), dec, 0.2)
        out, ns, ns_q, ns_s = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
        want = torch.tensor(case["expected"], dtype=torch.float32).reshape(out.shape)
        assert torch.equal(out.cpu(), want), case["cite"]
        assert (ns, ns_q, ns_s) == (0, 0.0, 0.0)  # BSI_PROFILE unset
        rows = ops.build_bsi_queries_cuda_batch(q.cuda(), dec, 0.2)
        out2, *_ = ops.batch_dot_product_multiquery_cuda_caps(rows, kcap)
        assert torch.equal(out2, out)


@pytest.mark.parametrize("layout", ["tiled", "canonical"])
@pytest.mark.parametrize("core", ["mfma", "valu"])
def test_ops_pipeline_matches_oracle_c1(ops, oracle, monkeypatch, layout, core):
    monkeypatch.setenv("BSI_KEY_LAYOUT", layout)
    monkeypatch.setenv("BSI_DOT_CORE", core)
    ops._reset_flag_cache()
    torch.manual_seed(123)
    Q, R, D = 64, 256, 2048
    K = torch.randn(R, D) * 0.02
    X = torch.randn(Q, D)
    kcap, nbytes, nk, d, W = ops.build_bsi_keys_cuda(K, 2, 0.5)
    assert (nbytes, nk, d, W) == (R * 6 * 32 * 8, R, D, 32)
    qcap = ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.5)
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    ints, out_dbg = ops.debug_chunk_ints(qcap, kcap, core)
    qb, kb = oracle.build_queries(X.numpy()), oracle.build_keys(K.numpy())
    want_ints, want_out = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    np.testing.assert_array_equal(host_u64(qcap.words), qb["words"])
    np.testing.assert_array_equal(qcap.chunk_scales.cpu().numpy(), qb["scales"])
    np.testing.assert_array_equal(kcap.slice_weights.cpu().numpy(), kb["slice_weights"])
    np.testing.assert_array_equal(qcap.slice_weights.cpu().numpy(), np.tile(oracle.slice_weights(7), (Q, 1)))
    np.testing.assert_array_equal(ints.cpu().numpy(), want_ints)
    np.testing.assert_array_equal(out.cpu().numpy(), want_out)
    np.testing.assert_array_equal(out_dbg.cpu().numpy(), want_out)
    # accuracy against the dense product: a statistical bound (keys sit on a 0.01 grid)
    dense = X.double() @ K.double().T
    rel = float(torch.linalg.norm(out.cpu().double() - dense) / torch.linalg.norm(dense))
    assert rel < 0.25, rel
    stats = ops.bsi_keys_cuda_stats(kcap)
    assert stats == {"W": 32, "d": D, "num_keys": R, "decimals": 2, "threshold": 0.5, "Sb_counts": {6: R}}
    rows = ops.build_bsi_queries_cuda_batch(X[:5].cuda(), 2, 0.5)
    assert ops.bsi_query_caps_stats(rows) == {"Q": 5, "W": 32, "S_counts": {7: 5}}


def test_ops_profile_flag_and_errors(ops, monkeypatch):
    monkeypatch.setenv("BSI_PROFILE", "1")
    ops._reset_flag_cache()
    K = torch.randn(64, 512)
    X = torch.randn(8, 512).cuda()
    kcap, *_ = ops.build_bsi_keys_cuda(K, 2)
    qcap = ops.build_bsi_queries_cuda_batch_packed(X, 2)
    q_ns, p_ns, t_ns = ops.get_last_query_build_profile_cuda()
    assert t_ns > 0 and t_ns == q_ns + p_ns
    out, ns, ns_q, ns_s = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    assert ns > 0 and ns_q == ns / 8 and ns_s == ns / (8 * 64)
    ops.reset_last_query_build_profile_cuda()
    assert ops.get_last_query_build_profile_cuda() == (0, 0, 0)
    q_bad = ops.build_bsi_queries_cuda_batch_packed(torch.randn(8, 256).cuda(), 2)
    with pytest.raises(RuntimeError, match="Word count mismatch"):
        ops.batch_dot_product_multiquery_cuda_batch_caps(q_bad, kcap)
    q_dec = ops.build_bsi_queries_cuda_batch_packed(X, 3)
    with pytest.raises(RuntimeError, match="Decimal mismatch"):
        ops.batch_dot_product_multiquery_cuda_batch_caps(q_dec, kcap)
    qcap.chunk_scales = qcap.chunk_scales[:, :1].contiguous()
    with pytest.raises(RuntimeError, match="Chunk scale stride mismatch"):
        ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)


def test_linear_drop_in(ops, oracle):
    from bsipytorch_amd.linear import BSIQuantizedLinear, quantize_model_bsi, sum_bsi_dot_query_vectors

    torch.manual_seed(0)
    lin = torch.nn.Linear(512, 192, bias=True)
    blin = BSIQuantizedLinear(lin, decimalPlaces=2, compress_threshold=0.5)
    x = torch.randn(2, 9, 512)
    y = blin(x.cuda())
    assert y.shape == (2, 9, 192) and y.dtype == x.dtype and y.is_cuda
    # the layer is exactly: BSI dot of the quantised activations and weights, plus the bias
    qb = oracle.build_queries(x.reshape(18, 512).numpy())
    kb = oracle.build_keys(lin.weight.detach().numpy())
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    want = torch.from_numpy(want) + lin.bias.detach()
    assert torch.equal(y.cpu().reshape(18, 192), want)
    # and close to the dense layer built from the de-quantised operands
    a = torch.from_numpy(qb["ints"] * np.repeat(qb["scales"], 256, axis=1) / 100.0)
    b = torch.from_numpy(kb["ints"] * kb["scales"][:, None] / 100.0)
    dense = (a @ b.T).float() + lin.bias.detach()
    assert torch.allclose(y.cpu().reshape(18, 192), dense, rtol=1e-4, atol=1e-5)
    # half-precision activations go in natively and come back in their dtype
    y16 = blin(x.cuda().to(torch.bfloat16))
    assert y16.dtype == torch.bfloat16 and y16.shape == (2, 9, 192)
    y2d = blin(x.cuda().reshape(18, 512))
    assert y2d.shape == (18, 192) and torch.equal(y2d, y.reshape(18, 192))
    assert blin.dot_calls == 3 and blin.dot_query_vectors_total == 54
    assert blin.weight_bsi_memory_bytes == 192 * 6 * 8 * 8 and blin.dot_ns_total == 0

    # layers fed the same tensor share one query build; an in-place change of the tensor forces a new one
    lin2 = torch.nn.Linear(512, 64, bias=False)
    blin2 = BSIQuantizedLinear(lin2, decimalPlaces=2, compress_threshold=0.5)
    xs = x.cuda().reshape(18, 512).contiguous()
    b0, b1 = blin.build_calls, blin2.build_calls
    ya, yb = blin(xs), blin2(xs)
    assert blin.build_calls == b0 + 1 and blin2.build_calls == b1  # second layer reused the planes
    kb2 = oracle.build_keys(lin2.weight.detach().numpy())
    _, want2 = oracle.dot_fixed(qb["words"], qb["scales"], kb2["words"], kb2["scales"], oracle.scale_inv(2, 2))
    assert torch.equal(yb.cpu(), torch.from_numpy(want2)) and torch.equal(ya, y.reshape(18, 192))
    xs.mul_(2.0)
    yc = blin2(xs)
    assert blin2.build_calls == b1 + 1 and not torch.equal(yc, yb)
    blin.dot_calls -= 1  # keep the call accounting below as it was

    class Tiny(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj = torch.nn.Linear(256, 256)
            self.fc1 = torch.nn.Linear(256, 512)
            self.lm_head = torch.nn.Linear(512, 100)

        def forward(self, t):
            return self.lm_head(torch.relu(self.fc1(self.q_proj(t))))

    m = Tiny()
    inp = torch.randn(3, 256)
    dense = m(inp)
    quantize_model_bsi(m, decimalPlaces=2, scope="all", compress_threshold=0.5, verbose=False)
    assert isinstance(m.q_proj, BSIQuantizedLinear) and isinstance(m.fc1, BSIQuantizedLinear)
    assert isinstance(m.lm_head, torch.nn.Linear)
    m.cuda()
    got = m(inp.cuda()).detach().cpu()
    cos = float((got * dense.detach()).sum() / (torch.linalg.norm(got) * torch.linalg.norm(dense.detach())))
    assert cos > 0.9, cos
    assert sum_bsi_dot_query_vectors(m) == 6
    m2 = Tiny()
    quantize_model_bsi(m2, scope="mlp", verbose=False)
    assert isinstance(m2.fc1, BSIQuantizedLinear) and isinstance(m2.q_proj, torch.nn.Linear)


# ------------------------------------------------------------------ decimal mode (slice count from the data)


def _decimal_case(Q, R, d, seed, qscale=1.0, kscale=0.5):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((Q, d)) * qscale).astype(np.float32)
    k = (rng.standard_normal((R, d)) * kscale).astype(np.float32)
    if Q > 1:
        x[1] = np.abs(x[1])  # a row without negatives: unsigned weights
    if R > 2:
        k[2] = 0.0
    return x, k


@pytest.mark.parametrize("Q,d,scale", [(9, 700, 1.0), (3, 64, 1.0e6), (70, 2048, 3.0), (2, 5, 1.0e15)])
def test_decimal_stats_and_pack_match_oracle(hip, oracle, Q, d, scale):
    L = hip.lib
    x, _ = _decimal_case(Q, 1, d, seed=Q + d, qscale=scale)
    want = oracle.build_decimal(x, 2)
    xd = torch.from_numpy(x).cuda()
    ints = torch.empty((Q, d), dtype=torch.int64, device="cuda")
    hip.check(L.bsi_hip_quantize_round_to_int64(xd.data_ptr(), hip.DTYPE_F32, Q * d, 100.0, ints.data_ptr(), st()), "round")
    max_abs = torch.full((1,), -5, dtype=torch.int64, device="cuda")   # must be cleared by the call
    neg = torch.full((Q,), 7, dtype=torch.int32, device="cuda")
    hip.check(L.bsi_hip_decimal_stats(ints.data_ptr(), Q, d, max_abs.data_ptr(), neg.data_ptr(), st()), "stats")
    assert np.array_equal(ints.cpu().numpy(), want["ints"])
    m = int(max_abs.item())
    assert m == int(np.abs(want["ints"]).max())
    assert np.array_equal(neg.cpu().numpy().astype(bool), want["negative"])
    S = oracle.choose_total_slices(m != 0, m)
    assert S == want["S"]
    W = (d + 63) // 64
    words = torch.full((Q, S, W), -1, dtype=torch.int64, device="cuda")
    hip.check(L.bsi_hip_pack_bits_batch(ints.data_ptr(), Q, d, S, W, words.data_ptr(), st()), "pack")
    assert np.array_equal(host_u64(words), want["words"])
    # all-zero batch: max 0, no negatives
    z = torch.zeros((4, 100), dtype=torch.int64, device="cuda")
    negz = torch.full((4,), 7, dtype=torch.int32, device="cuda")
    hip.check(L.bsi_hip_decimal_stats(z.data_ptr(), 4, 100, max_abs.data_ptr(), negz.data_ptr(), st()), "stats")
    assert int(max_abs.item()) == 0 and not negz.any()


def _run_weighted(hip, a, b, Q, R, W, layout=0, key_indices=None, R_total=None, scale_inv=1e-4):
    L = hip.lib
    A, Aw = dev(a["words"]), dev(a["slice_weights"])
    B, Bw = dev(b["words"]), dev(b["slice_weights"])
    Sa, Sb = a["words"].shape[1], b["words"].shape[1]
    if layout == 1:
        chunks = (W + 3) // 4
        Bt = torch.full((((R + 15) // 16) * chunks * Sb * 64,), -1, dtype=torch.int64, device="cuda")
        hip.check(L.bsi_hip_tile_key_planes(B.data_ptr(), R, Sb, W, Bt.data_ptr(), st()), "tile")
        B = Bt
    R_total = R if R_total is None else R_total
    out = torch.full((Q, R_total), float("nan"), dtype=torch.float32, device="cuda")
    idx = None if key_indices is None else torch.from_numpy(np.asarray(key_indices, dtype=np.int64)).cuda()
    hip.check(L.bsi_hip_dot_weighted(A.data_ptr(), Aw.data_ptr(), Sa, W, B.data_ptr(), layout, Bw.data_ptr(), Sb, R, Q,
                                     idx.data_ptr() if idx is not None else None, float(np.float32(scale_inv)), R_total,
                                     out.data_ptr(), st()), "weighted dot")
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("Q,R,d,qscale,layout", [(5, 7, 300, 1.0, 0), (33, 70, 2048, 1.0, 0), (64, 256, 2048, 1.0, 1),
                                                 (40, 33, 700, 1.0, 1), (3, 50, 640, 3.0e4, 0), (17, 40, 512, 1.0e9, 0),
                                                 (1, 1, 64, 1.0, 0), (32, 32, 512, 1.0, 0)])
def test_dot_weighted_matches_oracle(hip, oracle, Q, R, d, qscale, layout):
    """Decimal operands on both sides; large magnitudes take the narrow-step instantiation (Sa + Sb > 28).
    Bit-exact against the oracle's exact sum, which is also the integer matrix product of the rounded values."""
    x, k = _decimal_case(Q, R, d, seed=Q * 31 + R, qscale=qscale)
    a, b = oracle.build_decimal(x, 2), oracle.build_decimal(k, 2)
    W = (d + 63) // 64
    want = oracle.dot_weighted(a["words"], a["slice_weights"], b["words"], b["slice_weights"], np.float32(1e-4))
    got = _run_weighted(hip, a, b, Q, R, W, layout=layout)
    assert np.array_equal(got, want)
    exact = (a["ints"].astype(object) @ b["ints"].astype(object).T)
    if max(abs(int(v)) for v in exact.reshape(-1)) < 2 ** 53:
        assert np.array_equal(got, exact.astype(np.float64).astype(np.float32) * np.float32(1e-4))
    np.testing.assert_allclose(got, want, rtol=FP32_RTOL)  # the stated bar


def test_dot_weighted_key_indices_and_row_stride(hip, oracle):
    """Keys of one slice-count group scattered into a wider output by key_indices; other columns untouched."""
    Q, R, d, R_total = 10, 37, 300, 50
    x, k = _decimal_case(Q, R, d, seed=5)
    a, b = oracle.build_decimal(x, 2), oracle.build_decimal(k, 2)
    perm = np.random.default_rng(1).permutation(R_total)[:R]
    want = oracle.dot_weighted(a["words"], a["slice_weights"], b["words"], b["slice_weights"], np.float32(1e-4))
    got = _run_weighted(hip, a, b, Q, R, 5, key_indices=perm, R_total=R_total)
    assert np.array_equal(got[:, perm], want)
    untouched = np.setdiff1d(np.arange(R_total), perm)
    assert np.isnan(got[:, untouched]).all()


def test_dot_weighted_mixed_with_fixed_bit_keys(hip, oracle):
    x, k = _decimal_case(20, 45, 1024, seed=9, kscale=3.0)
    a, b = oracle.build_decimal(x, 2), oracle.build_keys(k, 2, 6)
    want = oracle.dot_weighted(a["words"], a["slice_weights"], b["words"], b["slice_weights"], np.float32(1e-4))
    for layout in (0, 1):
        assert np.array_equal(_run_weighted(hip, a, b, 20, 45, 16, layout=layout), want)


def test_dot_weighted_rejects_bad_arguments(hip):
    L = hip.lib
    t = torch.zeros((64,), dtype=torch.int64, device="cuda")
    f = torch.zeros((64,), dtype=torch.float32, device="cuda")
    assert L.bsi_hip_dot_weighted(t.data_ptr(), f.data_ptr(), 65, 1, t.data_ptr(), 0, f.data_ptr(), 2, 1, 1, None, 1.0, 1,
                                  f.data_ptr(), st()) != 0
    assert b"slice counts" in L.bsi_hip_last_error()
    assert L.bsi_hip_dot_weighted(t.data_ptr(), f.data_ptr(), 2, 1, t.data_ptr(), 2, f.data_ptr(), 2, 1, 1, None, 1.0, 1,
                                  f.data_ptr(), st()) != 0
    assert L.bsi_hip_dot_weighted(None, f.data_ptr(), 2, 1, t.data_ptr(), 0, f.data_ptr(), 2, 1, 1, None, 1.0, 1,
                                  f.data_ptr(), st()) != 0


def test_ops_decimal_mode_known_answers_and_pipeline(ops, oracle, monkeypatch):
    """BSI_FIXED_BITS=0: the reference's decimal API end to end (its check scripts' known answers), then a random
    batch against the oracle, the row-handle form, the 1-D builders and the keyset statistics."""
    monkeypatch.setenv("BSI_FIXED_BITS", "0")
    ops._reset_flag_cache()
    kat = json.load(open(GOLDEN))
    for case in kat["vector_dot"] + kat["batch_dot"]:
        q = torch.tensor(case["q"] if "K" in case else [case["q"]], dtype=torch.float32)
        K = torch.tensor(case["K"] if "K" in case else [case["k"]], dtype=torch.float32)
        dec = case["decimal_places"]
        kcap, *_ = ops.build_bsi_keys_cuda(K, dec, 0.2)
        qcap = ops.build_bsi_queries_cuda_batch_packed(q.cuda(), dec, 0.2)
        out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
        want = torch.tensor(case["expected"], dtype=torch.float32).reshape(out.shape)
        assert torch.allclose(out.cpu(), want, atol=1e-5), case["cite"]
    x, k = _decimal_case(33, 70, 2048, seed=3)
    a, b = oracle.build_decimal(x, 2), oracle.build_decimal(k, 2)
    want = oracle.dot_weighted(a["words"], a["slice_weights"], b["words"], b["slice_weights"], oracle.scale_inv(2, 2))
    kcap, nbytes, nk, d, W = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.2)
    assert (nk, d, W) == (70, 2048, 32) and nbytes == 70 * b["S"] * 32 * 8
    assert ops.bsi_keys_cuda_stats(kcap)["Sb_counts"] == {b["S"]: 70}
    qcap = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(x).cuda(), 2, 0.2)
    assert qcap.Sa == a["S"] and np.array_equal(host_u64(qcap.words), a["words"])
    assert np.array_equal(qcap.slice_weights.cpu().numpy(), a["slice_weights"])
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    assert np.array_equal(out.cpu().numpy(), want)
    rows = ops.build_bsi_queries_cuda_batch(torch.from_numpy(x).cuda(), 2, 0.2)
    out2, *_ = ops.batch_dot_product_multiquery_cuda_caps(rows, kcap)
    assert torch.equal(out2, out)
    assert ops.bsi_query_caps_stats(rows)["S_counts"] == {a["S"]: 33}
    # 1-D builders: the slice count follows that vector alone
    one = oracle.build_decimal(x[1:2], 2)
    h, mem, S, W1 = ops.build_bsi_query_cuda(torch.from_numpy(x[1]).cuda(), 2, 0.2)
    assert S == one["S"] and not h.twos_complement and np.array_equal(host_u64(h.dev_words), one["words"][0])
    hh, *_ = ops.build_bsi_query_cuda_hybrid(torch.from_numpy(x[0]).cuda(), 2, 0.5)
    assert hh.twos_complement
    want0 = oracle.build_decimal(x[0:1], 2)
    o0, *_ = ops.batch_dot_product_multiquery_cuda_caps([hh], kcap)
    assert np.array_equal(o0.cpu().numpy(), oracle.dot_weighted(want0["words"], want0["slice_weights"], b["words"],
                                                                 b["slice_weights"], oracle.scale_inv(2, 2)))
    with pytest.raises(RuntimeError, match="fixed-bit operands only"):
        ops.debug_chunk_ints(qcap, kcap)


def test_ops_decimal_queries_with_fixed_keys_and_the_reverse(ops, oracle, monkeypatch):
    x, k = _decimal_case(12, 40, 1024, seed=21, kscale=0.02)
    monkeypatch.setenv("BSI_FIXED_BITS_QUERIES", "0")
    ops._reset_flag_cache()
    a, b = oracle.build_decimal(x, 2), oracle.build_keys(k, 2, 6)
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.2)       # fixed 6-bit, tiled planes + int8 image
    qcap = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(x).cuda(), 2, 0.2)
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    assert np.array_equal(out.cpu().numpy(), oracle.dot_weighted(a["words"], a["slice_weights"], b["words"],
                                                                  b["slice_weights"], oracle.scale_inv(2, 2)))
    # the reverse: chunk-scaled fixed queries cannot meet decimal keys; row-scaled ones can
    monkeypatch.delenv("BSI_FIXED_BITS_QUERIES")
    monkeypatch.setenv("BSI_FIXED_BITS_KEYS", "0")
    ops._reset_flag_cache()
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.2)
    qcap = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(x).cuda(), 2, 0.2)
    with pytest.raises(RuntimeError, match="chunk-scaled queries need fixed-bit keys"):
        ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    monkeypatch.setenv("BSI_FIXED_CHUNK_SCALE", "0")
    ops._reset_flag_cache()
    qcap = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(x).cuda(), 2, 0.2)
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    qa, kb = oracle.build_queries(x, 2, 7), oracle.build_decimal(k, 2)
    ints, shifts, scales = oracle.quantize_fixed(x, 2, 7, False)
    aw = (oracle.slice_weights(7)[None, :] * scales[:, None]).astype(np.float32)
    want = oracle.dot_weighted(oracle.pack(ints, 7), aw, kb["words"], kb["slice_weights"], oracle.scale_inv(2, 2))
    assert np.array_equal(out.cpu().numpy(), want)


def test_linear_drop_in_decimal_mode(ops, monkeypatch):
    """BSIQuantizedLinear with BSI_FIXED_BITS=0: the output is the dense layer's up to the 10^-dec rounding grid."""
    from bsipytorch_amd import linear

    monkeypatch.setenv("BSI_FIXED_BITS", "0")
    ops._reset_flag_cache()
    torch.manual_seed(4)
    dense = torch.nn.Linear(512, 96).cuda()
    layer = linear.BSIQuantizedLinear(dense, decimalPlaces=3, compress_threshold=0.5)
    x = torch.randn(24, 512, device="cuda")
    with torch.no_grad():
        got, ref = layer(x), dense(x)
    # |error| <= sum over d of (|x| + |w| + grid) * grid / 2, far below this bound in practice
    assert (got - ref).abs().max().item() < 512 * 0.0005 * 5.0
    cos = torch.nn.functional.cosine_similarity(got.flatten(), ref.flatten(), dim=0).item()
    assert cos > 0.9999


# ------------------------------------------------------------------ keyset files


@pytest.mark.parametrize("mode", ["fixed-tiled", "fixed-canonical", "decimal"])
def test_keyset_file_round_trip(ops, oracle, monkeypatch, tmp_path, mode):
    """save_keyset_cuda / load_keyset_cuda: the planes on disk are the oracle's canonical planes, and the loaded
    keyset gives bit-identical dot outputs without re-quantising."""
    if mode == "fixed-canonical":
        monkeypatch.setenv("BSI_KEY_LAYOUT", "canonical")
    if mode == "decimal":
        monkeypatch.setenv("BSI_FIXED_BITS_KEYS", "0")
        monkeypatch.setenv("BSI_FIXED_CHUNK_SCALE", "0")
    ops._reset_flag_cache()
    R, d = 70, 1100  # ragged: 18 words per slice, 5 key tiles of 16
    rng = np.random.default_rng(8)
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    x = rng.standard_normal((40, d)).astype(np.float32)
    kcap, nbytes, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.5)
    want = oracle.build_decimal(k, 2) if mode == "decimal" else oracle.build_keys(k, 2, 6)
    assert np.array_equal(host_u64(ops.canonical_key_planes(kcap)), want["words"])
    written = ops.save_keyset_cuda(kcap, str(tmp_path / "layer"))
    mem, disk = ops.keyset_size_on_disk_cuda(kcap)
    assert written == disk and mem == nbytes == want["words"].size * 8
    assert disk < mem + R * want["words"].shape[1] * 4 + R * 4 + 1024
    loaded, nbytes2, nk, d2, W = ops.load_keyset_cuda(str(tmp_path / "layer"))
    assert (nbytes2, nk, d2, W) == (nbytes, R, d, 18)
    assert (loaded.Sb, loaded.decimals, loaded.fixed, loaded.layout) == (kcap.Sb, 2, kcap.fixed, kcap.layout)
    assert torch.equal(loaded.words, kcap.words) and torch.equal(loaded.slice_weights, kcap.slice_weights)
    if kcap.fixed:
        assert torch.equal(loaded.shifts, kcap.shifts) and torch.equal(loaded.ints8, kcap.ints8)
    qcap = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(x).cuda(), 2, 0.5)
    a, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    b, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, loaded)
    assert torch.equal(a, b)
    # damaged files are refused
    path = tmp_path / "layer" / "keyset.bsik"
    raw = path.read_bytes()
    path.write_bytes(raw[:-100])
    with pytest.raises(RuntimeError, match="truncated"):
        ops.load_keyset_cuda(str(tmp_path / "layer"))
    path.write_bytes(b"NOTAKEYS" + raw[8:])
    with pytest.raises(RuntimeError, match="not a BSI keyset file"):
        ops.load_keyset_cuda(str(tmp_path / "layer"))


def test_save_and_load_bsi_model(ops, tmp_path):
    from bsipytorch_amd import linear

    torch.manual_seed(2)

    def make():
        return torch.nn.Sequential(torch.nn.Linear(512, 256), torch.nn.ReLU(), torch.nn.Linear(256, 64, bias=False)).cuda()

    model = make()
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    x = torch.randn(33, 512, device="cuda")
    with torch.no_grad():
        want = model(x)
    meta = linear.save_bsi_model(model, str(tmp_path / "m"))
    assert [m["name"] for m in meta] == ["0", "2"] and meta[0]["has_bias"] and not meta[1]["has_bias"]
    saved = json.load(open(tmp_path / "m" / "manifest.json"))
    assert saved[0]["in"] == 512 and saved[0]["out"] == 256 and saved[0]["decimalPlaces"] == 2
    # 6 planes of 512 bits per row = 0.75 byte per weight, plus weights, shifts and the header
    assert saved[0]["keyset_bytes"] < 512 * 256 * 0.75 + 256 * 6 * 4 + 256 * 4 + 1024
    other = make()  # different random weights: the loaded layers must not depend on them
    linear.load_bsi_model(other, str(tmp_path / "m"))
    assert isinstance(other[0], linear.BSIQuantizedLinear) and other[0].weight_fp32 is None
    with torch.no_grad():
        got = other(x)
    assert torch.equal(got, want)


# ------------------------------------------------------------------ empty and degenerate inputs


@pytest.mark.parametrize("bits", ["fixed", "decimal"])
def test_empty_and_degenerate_inputs(ops, hip, monkeypatch, bits):
    """Zero rows, zero columns, a single element: builders return well-formed handles, the dot refuses empty
    operands with the reference's messages (bsi_cuda.cpp:672-682), and the raw entry points accept zero sizes."""
    if bits == "decimal":
        monkeypatch.setenv("BSI_FIXED_BITS", "0")
        ops._reset_flag_cache()
    L = hip.lib
    kcap, nbytes, nk, d, W = ops.build_bsi_keys_cuda(torch.randn(5, 64), 2, 0.2)
    q0 = ops.build_bsi_queries_cuda_batch_packed(torch.zeros((0, 64)).cuda(), 2, 0.2)
    assert q0.Q == 0 and q0.words.shape[0] == 0 and q0.W == 1
    with pytest.raises(RuntimeError, match="Empty query batch"):
        ops.batch_dot_product_multiquery_cuda_batch_caps(q0, kcap)
    k0, nb0, nk0, d0, W0 = ops.build_bsi_keys_cuda(torch.zeros((0, 64)), 2, 0.2)
    assert (nb0, nk0, d0, W0) == (0, 0, 64, 1)
    q1 = ops.build_bsi_queries_cuda_batch_packed(torch.randn(3, 64).cuda(), 2, 0.2)
    with pytest.raises(RuntimeError, match="Empty keys"):
        ops.batch_dot_product_multiquery_cuda_batch_caps(q1, k0)
    with pytest.raises(RuntimeError, match="Empty keys or queries"):
        ops.batch_dot_product_multiquery_cuda_caps([], kcap)
    # one element per row
    k1, *_ = ops.build_bsi_keys_cuda(torch.tensor([[0.25], [-0.5]]), 2, 0.2)
    qq = ops.build_bsi_queries_cuda_batch_packed(torch.tensor([[2.0], [-1.0], [0.0]]).cuda(), 2, 0.2)
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qq, k1)
    assert torch.allclose(out.cpu(), torch.tensor([[0.5, -1.0], [-0.25, 0.5], [0.0, 0.0]]), atol=1e-6)
    # all-zero operands
    kz, *_ = ops.build_bsi_keys_cuda(torch.zeros((4, 256)), 2, 0.2)
    qz = ops.build_bsi_queries_cuda_batch_packed(torch.zeros((2, 256)).cuda(), 2, 0.2)
    out, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qz, kz)
    assert not out.any() and out.shape == (2, 4)
    # raw entry points: zero sizes are accepted without touching the pointers
    assert L.bsi_hip_build_fixed(None, hip.DTYPE_F32, 0, 64, 2, 7, 1, 0.0, None, None, None, None, st()) == 0
    assert L.bsi_hip_pack_bits_batch(None, 0, 64, 7, 1, None, st()) == 0
    assert L.bsi_hip_dot(None, None, None, 1, 7, 1, None, 0, None, 6, 0, 4, 1.0, 0, None, None, 0, None, 0, st()) == 0
    assert L.bsi_hip_dot_weighted(None, None, 7, 1, None, 0, None, 6, 0, 4, None, 1.0, 0, None, st()) == 0
    m = torch.full((1,), 9, dtype=torch.int64, device="cuda")
    assert L.bsi_hip_decimal_stats(None, 0, 64, m.data_ptr(), None, st()) == 0 and int(m.item()) == 0


# ------------------------------------------------------------------ decimal mode on the matrix cores


def _image_order(a: np.ndarray, chunks: int) -> np.ndarray:
    """[..., d] values -> [..., chunks*256] in the int8 images' element order (element 32w + 8m + t of a chunk at
    byte 32w + 4t + m), zero padded."""
    d = a.shape[-1]
    padded = np.zeros(a.shape[:-1] + (chunks * 256,), dtype=np.int64)
    padded[..., :d] = a
    e = np.arange(chunks * 256)
    pos = (e // 32) * 32 + ((e % 32) % 8) * 4 + (e % 32) // 8
    out = np.zeros_like(padded)
    out[..., pos] = padded
    return out


def _digits_dev(hip, words: np.ndarray):
    rows, S, W = words.shape
    chunks = (W + 3) // 4
    out = torch.full(((S + 6) // 7, rows, chunks * 256), 77, dtype=torch.int8, device="cuda")
    words_d = dev(words)  # named, so that it lives until the kernel has run
    hip.check(hip.lib.bsi_hip_planes_to_int8_digits(words_d.data_ptr(), rows, S, W, out.data_ptr(), st()), "digits")
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("Q,d,scale", [(9, 700, 1.0), (3, 64, 1.0e6), (33, 2048, 3.0), (2, 5, 1.0e15), (4, 256, 0.0)])
def test_digit_images_match_oracle(hip, oracle, Q, d, scale):
    x, _ = _decimal_case(Q, 1, d, seed=Q + d, qscale=scale)
    b = oracle.build_decimal(x, 2)
    got = _digits_dev(hip, b["words"]).cpu().numpy().astype(np.int64)
    want = _image_order(oracle.int8_digits(b["ints"], b["S"]), (b["words"].shape[2] + 3) // 4)
    assert got.shape == want.shape and np.array_equal(got, want)


def _run_digits(hip, a_dig, aw, Sa, k_dig, preshift, bw, Sb, W, Q, R, key_indices=None, R_total=None, bias=None,
                k_tiled=0):
    L = hip.lib
    nq, nk = a_dig.shape[0], (1 if k_tiled else k_dig.shape[0])
    R_total = R if R_total is None else R_total
    out = torch.full((Q, R_total), float("nan"), dtype=torch.float32, device="cuda")
    nbytes = int(L.bsi_hip_dot_digits_workspace_bytes(Q, nq, R, nk))
    assert nbytes == nq * Q * nk * R * 4
    ws = torch.empty((nbytes,), dtype=torch.uint8, device="cuda")
    idx = None if key_indices is None else torch.from_numpy(np.asarray(key_indices, dtype=np.int64)).cuda()
    Aw, Bw = dev(aw), dev(bw)
    hip.check(L.bsi_hip_dot_digits(a_dig.data_ptr(), nq, Aw.data_ptr(), Sa, k_dig.data_ptr(), nk, preshift, Bw.data_ptr(),
                                   Sb, W, R, Q, idx.data_ptr() if idx is not None else None, float(np.float32(1e-4)),
                                   R_total, bias.data_ptr() if bias is not None else None, out.data_ptr(), ws.data_ptr(),
                                   nbytes, k_tiled, st()), "digit dot")
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("tile", [0, 128, 12864, 64, 6432])
@pytest.mark.parametrize("Q,R,d,qscale", [(5, 7, 300, 1.0), (70, 150, 2048, 1.0), (64, 256, 2048, 30.0),
                                          (17, 40, 512, 1.0e6), (1, 33, 8192, 1.0)])
def test_dot_digits_matches_oracle(hip, oracle, Q, R, d, qscale, tile):
    """Decimal operands as int8 digits through the int32-sum mode of the MFMA kernel (every tile): bit-identical
    to the oracle's exact weighted-slice sum, i.e. to the integer matrix product of the rounded values."""
    x, k = _decimal_case(Q, R, d, seed=Q * 31 + R, qscale=qscale)
    a, b = oracle.build_decimal(x, 2), oracle.build_decimal(k, 2)
    W = (d + 63) // 64
    want = oracle.dot_weighted(a["words"], a["slice_weights"], b["words"], b["slice_weights"], np.float32(1e-4))
    hip.check(hip.lib.bsi_hip_set_option(hip.OPT_I8_TILE, tile), "opt")
    try:
        for route in (1, 2, 0):  # stacked digits + combine pass; digits recombined in the accumulator; by cost
            hip.check(hip.lib.bsi_hip_set_option(hip.OPT_DIGITS_ROUTE, route), "opt")
            got = _run_digits(hip, _digits_dev(hip, a["words"]), a["slice_weights"], a["S"], _digits_dev(hip, b["words"]),
                              0, b["slice_weights"], b["S"], W, Q, R)
            assert np.array_equal(got, want), route
    finally:
        hip.check(hip.lib.bsi_hip_set_option(hip.OPT_I8_TILE, 0), "opt")
        hip.check(hip.lib.bsi_hip_set_option(hip.OPT_DIGITS_ROUTE, 0), "opt")
    exact = a["ints"].astype(object) @ b["ints"].astype(object).T
    if max(abs(int(v)) for v in exact.reshape(-1)) < 2 ** 53:
        assert np.array_equal(got, exact.astype(np.float64).astype(np.float32) * np.float32(1e-4))


def test_dot_digits_fixed_images_indices_bias_and_stride(hip, oracle):
    """Fixed-bit key image (one digit pre-shifted by 8 - Sb) under decimal queries, and a row-scaled fixed query
    image against decimal keys; key_indices scatter into a wider output; the bias is added after the scale."""
    Q, R, d, W = 20, 45, 1024, 16
    x, k = _decimal_case(Q, R, d, seed=9, kscale=3.0)
    a, b = oracle.build_decimal(x, 2), oracle.build_keys(k, 2, 6)
    want = oracle.dot_weighted(a["words"], a["slice_weights"], b["words"], b["slice_weights"], np.float32(1e-4))
    k8 = torch.empty((1, R, 4 * 256), dtype=torch.int8, device="cuda")
    _src1 = dev(b["words"])  # named, so that it lives until the kernel has run
    hip.check(hip.lib.bsi_hip_planes_to_int8(_src1.data_ptr(), R, 6, W, k8.data_ptr(), st()), "image")
    a_dig = _digits_dev(hip, a["words"])
    perm = np.random.default_rng(3).permutation(60)[:R]
    bias = torch.randn(R, device="cuda")
    k8t = torch.full((int(hip.lib.bsi_hip_int8_tiled_bytes(R, W)),), 77, dtype=torch.int8, device="cuda")
    _src2 = dev(b["words"])  # named, so that it lives until the kernel has run
    hip.check(hip.lib.bsi_hip_planes_to_int8_tiled(_src2.data_ptr(), R, 6, W, k8t.data_ptr(), st()), "image")
    for route in (1, 2):
        hip.check(hip.lib.bsi_hip_set_option(hip.OPT_DIGITS_ROUTE, route), "opt")
        got = _run_digits(hip, a_dig, a["slice_weights"], a["S"], k8, 2, b["slice_weights"], 6, W, Q, R)
        assert np.array_equal(got, want), route
        got = _run_digits(hip, a_dig, a["slice_weights"], a["S"], k8t, 2, b["slice_weights"], 6, W, Q, R, k_tiled=1)
        assert np.array_equal(got, want), route
        got = _run_digits(hip, a_dig, a["slice_weights"], a["S"], k8, 2, b["slice_weights"], 6, W, Q, R, key_indices=perm,
                          R_total=60, bias=bias)
        assert np.array_equal(got[:, perm], want + bias.cpu().numpy()[None, :]), route
        assert np.isnan(got[:, np.setdiff1d(np.arange(60), perm)]).all()
    hip.check(hip.lib.bsi_hip_set_option(hip.OPT_DIGITS_ROUTE, 0), "opt")
    # the reverse: 7-bit row-scaled queries (image pre-shifted by 1) against decimal keys
    ints, shifts, scales = oracle.quantize_fixed(x, 2, 7, False)
    aw = (oracle.slice_weights(7)[None, :] * scales[:, None]).astype(np.float32)
    kb = oracle.build_decimal(k, 2)
    want = oracle.dot_weighted(oracle.pack(ints, 7), aw, kb["words"], kb["slice_weights"], np.float32(1e-4))
    q8 = torch.empty((1, Q, 4 * 256), dtype=torch.int8, device="cuda")
    _src3 = dev(oracle.pack(ints, 7))  # named, so that it lives until the kernel has run
    hip.check(hip.lib.bsi_hip_planes_to_int8(_src3.data_ptr(), Q, 7, W, q8.data_ptr(), st()), "image")
    got = _run_digits(hip, q8, aw, 7, _digits_dev(hip, kb["words"]), 1, kb["slice_weights"], kb["S"], W, Q, R)
    assert np.array_equal(got, want)


def test_ops_decimal_mfma_and_popcount_routes_agree(ops, monkeypatch):
    """BSI_DECIMAL_MFMA=0 keeps decimal operands on the popcount kernel; both routes give the same bits."""
    torch.manual_seed(6)
    X, K = torch.randn(70, 2048), torch.randn(150, 2048) * 0.02
    outs = {}
    for flag in ("1", "0"):
        monkeypatch.setenv("BSI_FIXED_BITS", "0")
        monkeypatch.setenv("BSI_DECIMAL_MFMA", flag)
        ops._reset_flag_cache()
        kcap, *_ = ops.build_bsi_keys_cuda(K, 2, 0.2)
        qcap = ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.2)
        assert (qcap.digits8 is not None) == (flag == "1") and (kcap.digits8 is not None) == (flag == "1")
        outs[flag], *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
        rows = ops.build_bsi_queries_cuda_batch(X.cuda(), 2, 0.2)
        o2, *_ = ops.batch_dot_product_multiquery_cuda_caps(rows, kcap)
        assert torch.equal(o2, outs[flag])
    assert torch.equal(outs["0"], outs["1"])
    dense = (X.double() @ K.double().T).float().cuda()
    assert (outs["1"] - dense).abs().max().item() < 2048 * 0.005 * 4.0


@pytest.mark.parametrize("R,d", [(64, 256), (150, 2048), (1, 64), (200, 700)])
def test_tiled_key_image_holds_the_row_major_bytes(hip, oracle, R, d):
    """[ceil(R/64)][2 chunks][64][128]: half-chunk h of row r sits at tile r // 64, block h, row r % 64; padding rows
    are zero."""
    rng = np.random.default_rng(R)
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    kb = oracle.build_keys(k, 2, 6)
    W = (d + 63) // 64
    chunks = (W + 3) // 4
    words = dev(kb["words"])
    rows = torch.empty((R, chunks * 256), dtype=torch.int8, device="cuda")
    hip.check(hip.lib.bsi_hip_planes_to_int8(words.data_ptr(), R, 6, W, rows.data_ptr(), st()), "rows")
    nbytes = int(hip.lib.bsi_hip_int8_tiled_bytes(R, W))
    tiles = (R + 63) // 64
    assert nbytes == tiles * chunks * 2 * 8192
    tiled = torch.full((nbytes,), 77, dtype=torch.int8, device="cuda")
    hip.check(hip.lib.bsi_hip_planes_to_int8_tiled(words.data_ptr(), R, 6, W, tiled.data_ptr(), st()), "tiled")
    t = tiled.view(tiles, chunks * 2, 64, 128).permute(0, 2, 1, 3).reshape(tiles * 64, chunks * 256)
    assert torch.equal(t[:R], rows) and not t[R:].any()


def test_warm_hint_changes_nothing_but_the_cache(ops, oracle):
    """bsi_hip_dot_bias_warm: same bits as without the hint, for every tile, with and without a bias; the warmed
    region is only read."""
    rng = np.random.default_rng(12)
    Q, R, d = 70, 150, 2048
    x = rng.standard_normal((Q, d)).astype(np.float32)
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    kcap, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.5)
    other, *_ = ops.build_bsi_keys_cuda(torch.from_numpy(k[::-1].copy()), 2, 0.5)
    before = other.ints8.clone()
    qcap = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(x).cuda(), 2, 0.5)
    bias = torch.randn(R, device="cuda")
    from bsipytorch_amd import _lib
    for tile in (0, 128, 12864, 64, 6432):
        _lib.check(_lib.lib.bsi_hip_set_option(_lib.OPT_I8_TILE, tile), "opt")
        for b in (None, bias):
            plain, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap, b)
            warm, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap, b, other)
            assert torch.equal(plain, warm), (tile, b is not None)
    _lib.check(_lib.lib.bsi_hip_set_option(_lib.OPT_I8_TILE, 0), "opt")
    assert torch.equal(other.ints8, before)
    # few query rows stream the planes; the hint is accepted there too
    q1 = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(x[:3]).cuda(), 2, 0.5)
    a, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(q1, kcap)
    b2, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(q1, kcap, None, other)
    assert torch.equal(a, b2)


def test_quantized_model_links_layers_for_the_warm_hint(ops, monkeypatch):
    from bsipytorch_amd import linear

    torch.manual_seed(3)
    model = torch.nn.Sequential(torch.nn.Linear(256, 128), torch.nn.ReLU(), torch.nn.Linear(128, 256),
                                torch.nn.ReLU(), torch.nn.Linear(256, 64)).cuda()
    x = torch.randn(40, 256, device="cuda")
    monkeypatch.setenv("BSI_WARM_NEXT", "0")
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    assert all(m.__dict__["_next_bsi_layer"] is None for m in model if isinstance(m, linear.BSIQuantizedLinear))
    with torch.no_grad():
        want = model(x)
    monkeypatch.setenv("BSI_WARM_NEXT", "1")
    assert linear.link_bsi_layers(model) == 3
    assert model[0].__dict__["_next_bsi_layer"] is model[2] and model[4].__dict__["_next_bsi_layer"] is model[0]
    with torch.no_grad():
        got = model(x)
    assert torch.equal(got, want)


def test_fused_sibling_layers_are_bit_identical(ops, oracle):
    """q_proj / k_proj / v_proj served by one dot over their stacked keys: same bits as three dots; keyset
    concatenation and row views keep every row's planes, weights and shifts."""
    from bsipytorch_amd import linear

    class Attn(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj = torch.nn.Linear(512, 128)
            self.k_proj = torch.nn.Linear(512, 128)
            self.v_proj = torch.nn.Linear(512, 192, bias=False)   # not all biased: members add their own
            self.out_proj = torch.nn.Linear(128, 512)

        def forward(self, x):
            return self.out_proj(self.q_proj(x) * self.k_proj(x)) + self.v_proj(x).sum(-1, keepdim=True)

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a, self.b = Attn(), Attn()

        def forward(self, x):
            return self.b(self.a(x))

    torch.manual_seed(5)
    model = Block().cuda()
    with torch.no_grad():
        model.b.v_proj.weight.mul_(3.0)
    x = torch.randn(2, 40, 512, device="cuda")
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    with torch.no_grad():
        want = model(x)
        want_q = model.a.q_proj(x)
    planes_before = [ops.canonical_key_planes(m._bsi_keys_cuda).clone() for m in (model.a.q_proj, model.a.k_proj, model.a.v_proj)]
    assert linear.fuse_sibling_layers(model) == 2
    g = model.a.q_proj.__dict__["_fused"][0]
    assert g.keys.num_keys == 128 + 128 + 192 and g.bias is None and g.next_layer is model.a.out_proj
    assert model.a.out_proj.__dict__["_next_bsi_layer"] is model.b.q_proj
    for m, before in zip((model.a.q_proj, model.a.k_proj, model.a.v_proj), planes_before):
        assert torch.equal(ops.canonical_key_planes(m._bsi_keys_cuda), before)
    with torch.no_grad():
        got = model(x)
        got_q = model.a.q_proj(x)
    assert torch.equal(got, want) and torch.equal(got_q, want_q) and got_q.shape == (2, 40, 128)
    # all members biased: the stacked bias goes into the dot
    torch.manual_seed(6)
    m2 = Attn().cuda()
    m2.v_proj = torch.nn.Linear(512, 192).cuda()
    linear.quantize_model_bsi(m2, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    with torch.no_grad():
        want2 = m2(x)
    linear.fuse_sibling_layers(m2)
    assert m2.q_proj.__dict__["_fused"][0].bias is not None
    with torch.no_grad():
        assert torch.equal(m2(x), want2)
    # a second, different input must not be served from the first one's result
    with torch.no_grad():
        y = m2(x * 2.0)
    assert not torch.equal(y, want2)


def test_model_harness_helpers(ops, capsys):
    """Error statistics, byte accounting and compression summary of a quantised model (the reference's harness
    helpers, verify_accuracy_bsi.py:282-432 and benchmark_performance_bsi.py:488-503)."""
    from bsipytorch_amd import linear

    torch.manual_seed(9)
    model = torch.nn.Sequential(torch.nn.Linear(256, 128), torch.nn.ReLU(), torch.nn.Linear(128, 64, bias=False)).cuda()
    dense_bytes = linear.get_model_static_bytes(model)
    assert dense_bytes == (256 * 128 + 128 + 128 * 64) * 4
    cfg = linear.build_layer_config(2, None, 3)
    assert cfg == {"default": 2, "mlp": 3} and linear.build_layer_config(2, None, None) == 2
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    summary = linear.summarize_bsi_model(model)
    assert summary["num_quantized_layers"] == 2 and summary["total_slices"] == (128 + 64) * 6
    assert summary["layers"][0]["weight_bsi_disk_bytes"] > 128 * 6 * 4 * 8
    assert linear.bsi_full_model_static_bytes(model, summary) == 128 * 4 + summary["total_bsi_bytes"]
    lines, overall = linear.compression_summary_lines(summary)
    assert len(lines) == 2 and overall == (0, (128 + 64) * 6, 0.0)
    linear.print_compression_summary(summary)
    assert "Overall compressed slices: 0/1152" in capsys.readouterr().out
    x = torch.randn(10, 256, device="cuda")
    linear.enable_bsi_error_stats(model, True)
    with torch.no_grad():
        model(x)
        model(x)
    stats = linear.collect_bsi_error_stats(model)
    assert len(stats) == 2 and all(s["samples_tracked"] == 20 for s in stats)
    assert all(s["cosine"] > 0.9 and s["mse"] >= 0 and s["max_abs"] > 0 for s in stats)
    assert stats[0]["mse"] >= stats[1]["mse"]
    linear.enable_bsi_error_stats(model, False)
    with torch.no_grad():
        model(x)
    assert linear.collect_bsi_error_stats(model)[0]["samples_tracked"] == 20


# ------------------------------------------------------------------ fused build + dot for a few rows


@pytest.mark.parametrize("Q", [1, 2, 3, 4])
@pytest.mark.parametrize("R,d,kind", [(200, 2048, "randn"), (33, 4096, "outliers"), (16400, 1024, "relu"), (75, 700 + 68, "ties")])
def test_linear_few_rows_matches_build_plus_dot(hip, oracle, Q, R, d, kind):
    """bsi_hip_linear_few_rows against the oracle's build + dot (so also against the two-launch path, which the
    other tests hold to the same oracle): one or two key tiles per workgroup, ragged D (768 = 3 chunks), a chunk of
    zeros, an outlier."""
    L = hip.lib
    x = _inputs(max(Q, 3), d, seed=Q * 13 + R, kind=kind)[:Q]
    rng = np.random.default_rng(R)
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    qb, kb = oracle.build_queries(x, 2, 7), oracle.build_keys(k, 2, 6)
    assert qb["chunk_scale"]
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    W = (d + 63) // 64
    chunks = W // 4
    B = dev(kb["words"])
    Bt = torch.full((((R + 15) // 16) * chunks * 6 * 64,), -1, dtype=torch.int64, device="cuda")
    hip.check(L.bsi_hip_tile_key_planes(B.data_ptr(), R, 6, W, Bt.data_ptr(), st()), "tile")
    Bw = dev(kb["slice_weights"])
    xd = torch.from_numpy(x).cuda()
    bias = torch.randn(R, device="cuda")
    for b in (None, bias):
        out = torch.full((Q, R + 3), float("nan"), dtype=torch.float32, device="cuda")
        hip.check(L.bsi_hip_linear_few_rows(xd.data_ptr(), hip.DTYPE_F32, Q, d, 2, 7, Bt.data_ptr(), Bw.data_ptr(), 6, R,
                                            float(oracle.scale_inv(2, 2)), R + 3, b.data_ptr() if b is not None else None,
                                            out.data_ptr(), st()), "fused")
        got = out.cpu().numpy()
        expect = want if b is None else want + b.cpu().numpy()[None, :]
        assert np.array_equal(got[:, :R], expect.astype(np.float32))
        assert np.isnan(got[:, R:]).all()


@pytest.mark.parametrize("dec", [0, 1, 3])
def test_linear_few_rows_other_decimal_places(hip, oracle, dec):
    """10^dec of 1 and 10 take the kernel's integer rounding route (as 100 does), 1000 its float64 route."""
    L = hip.lib
    Q, R, d = 3, 50, 1024
    x = _inputs(Q, d, seed=dec, kind="ties") * np.float32(10.0 ** (2 - dec))
    k = (np.random.default_rng(dec).standard_normal((R, d)) * (0.02 * 10.0 ** (2 - dec))).astype(np.float32)
    qb, kb = oracle.build_queries(x, dec, 7), oracle.build_keys(k, dec, 6)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(dec, dec), want_ints=False)
    Bt = torch.empty((4 * 4 * 6 * 64,), dtype=torch.int64, device="cuda")
    planes_d, x_d = dev(kb["words"]), torch.from_numpy(x).cuda()  # named, so that they live until the kernels have run
    hip.check(L.bsi_hip_tile_key_planes(planes_d.data_ptr(), R, 6, 16, Bt.data_ptr(), st()), "tile")
    Bw = dev(kb["slice_weights"])
    out = torch.empty((Q, R), dtype=torch.float32, device="cuda")
    hip.check(L.bsi_hip_linear_few_rows(x_d.data_ptr(), hip.DTYPE_F32, Q, d, dec, 7, Bt.data_ptr(),
                                        Bw.data_ptr(), 6, R, float(oracle.scale_inv(dec, dec)), R, None, out.data_ptr(),
                                        st()), "fused")
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)


def test_linear_few_rows_long_rows_and_lds_limit(hip, oracle):
    """Rows of 96 chunks: three of them fit the kernel's LDS query buffer and run in two passes over the chunk
    accumulators; four do not and are refused on the host."""
    L = hip.lib
    R, d = 20, 24576
    x = _inputs(4, d, seed=5, kind="outliers")
    x[0, 7] = 3.0e7   # x * 100 beyond 32 bits: that chunk takes the kernel's 64-bit route
    x[2, 20000] = -4.0e7  # and one among a wave's later items
    k = (np.random.default_rng(2).standard_normal((R, d)) * 0.02).astype(np.float32)
    qb, kb = oracle.build_queries(x[:3], 2, 7), oracle.build_keys(k, 2, 6)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    W = d // 64
    Bt = torch.empty((2 * (W // 4) * 6 * 64,), dtype=torch.int64, device="cuda")
    _src4 = dev(kb["words"])  # named, so that it lives until the kernel has run
    hip.check(L.bsi_hip_tile_key_planes(_src4.data_ptr(), R, 6, W, Bt.data_ptr(), st()), "tile")
    Bw = dev(kb["slice_weights"])
    xd = torch.from_numpy(x).cuda()
    out = torch.empty((4, R), dtype=torch.float32, device="cuda")
    hip.check(L.bsi_hip_linear_few_rows(xd.data_ptr(), hip.DTYPE_F32, 3, d, 2, 7, Bt.data_ptr(), Bw.data_ptr(), 6, R,
                                        float(oracle.scale_inv(2, 2)), R, None, out.data_ptr(), st()), "fused")
    assert np.array_equal(out[:3].cpu().numpy(), want)
    assert L.bsi_hip_linear_few_rows(xd.data_ptr(), hip.DTYPE_F32, 4, d, 2, 7, Bt.data_ptr(), Bw.data_ptr(), 6, R,
                                     float(oracle.scale_inv(2, 2)), R, None, out.data_ptr(), st()) != 0
    assert b"LDS query buffer" in L.bsi_hip_last_error()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_linear_few_rows_half_inputs_and_limits(hip, oracle, dtype):
    L = hip.lib
    torch.manual_seed(3)
    xh = (torch.randn(2, 1024) * 3).to(dtype)
    x = xh.to(torch.float32).numpy()
    k = (np.random.default_rng(1).standard_normal((40, 1024)) * 0.02).astype(np.float32)
    qb, kb = oracle.build_queries(x, 2, 7), oracle.build_keys(k, 2, 6)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    Bt = torch.empty((3 * 4 * 6 * 64,), dtype=torch.int64, device="cuda")
    _src5 = dev(kb["words"])  # named, so that it lives until the kernel has run
    hip.check(L.bsi_hip_tile_key_planes(_src5.data_ptr(), 40, 6, 16, Bt.data_ptr(), st()), "tile")
    Bw = dev(kb["slice_weights"])
    out = torch.empty((2, 40), dtype=torch.float32, device="cuda")
    xd = xh.cuda()
    code = hip.DTYPE_F16 if dtype == torch.float16 else hip.DTYPE_BF16
    hip.check(L.bsi_hip_linear_few_rows(xd.data_ptr(), code, 2, 1024, 2, 7, Bt.data_ptr(), Bw.data_ptr(), 6, 40,
                                        float(oracle.scale_inv(2, 2)), 40, None, out.data_ptr(), st()), "fused")
    assert np.array_equal(out.cpu().numpy(), want)
    # limits are refused on the host
    assert L.bsi_hip_linear_few_rows(xd.data_ptr(), code, 5, 1024, 2, 7, Bt.data_ptr(), Bw.data_ptr(), 6, 40, 1e-4, 40,
                                     None, out.data_ptr(), st()) != 0
    assert b"at most 4 query rows" in L.bsi_hip_last_error()
    assert L.bsi_hip_linear_few_rows(xd.data_ptr(), code, 2, 960, 2, 7, Bt.data_ptr(), Bw.data_ptr(), 6, 40, 1e-4, 40,
                                     None, out.data_ptr(), st()) != 0   # 15 words per slice: no chunk scales
    assert L.bsi_hip_linear_few_rows(xd.data_ptr(), code, 2, 1024, 2, 7, Bt.data_ptr(), Bw.data_ptr(), 5, 40, 1e-4, 40,
                                     None, out.data_ptr(), st()) != 0


@pytest.mark.parametrize("Q,R,d,with_bias", [(64, 200, 1024, True), (130, 75, 2048, False), (7, 33, 512, True), (33, 4100, 256, True)])
def test_linear_one_call_matches_build_plus_dot(hip, oracle, ops, Q, R, d, with_bias):
    """bsi_hip_linear (through bsi_ops.linear_cuda) against the oracle's build + dot, with and without the shared
    build (second call on the same tensor), with a changed input in between, and against the two-call path."""
    x = _inputs(Q, d, seed=Q + R, kind="outliers")
    k = (np.random.default_rng(R).standard_normal((R, d)) * 0.02).astype(np.float32)
    qb, kb = oracle.build_queries(x, 2, 7), oracle.build_keys(k, 2, 6)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    keys = ops.build_bsi_keys_cuda(torch.from_numpy(k), 2, 0.5)[0]
    bias = torch.randn(R, device="cuda") if with_bias else None
    expect = want if bias is None else want + bias.cpu().numpy()[None, :]
    xd = torch.from_numpy(x).cuda()
    ops.linear_cuda_forget()
    out1 = ops.linear_cuda(xd, keys, 2, bias)
    out2 = ops.linear_cuda(xd, keys, 2, bias)          # same tensor: the build is reused
    assert np.array_equal(out1.cpu().numpy(), expect.astype(np.float32)) and torch.equal(out1, out2)
    other = torch.from_numpy(_inputs(Q, d, seed=99)).cuda()
    ops.linear_cuda(other, keys, 2, bias)              # overwrites the workspace
    xd.mul_(1.0)                                       # same values, new version: rebuilt, same result
    assert torch.equal(ops.linear_cuda(xd, keys, 2, bias), out1)
    qcap = ops.build_bsi_queries_cuda_batch_packed(xd, 2, 0.5)
    two = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, keys, bias)[0]
    assert torch.equal(two, out1)


def test_layer_forward_one_call_path_and_graph_replay(ops, monkeypatch):
    """BSIQuantizedLinear takes the one-call path for ordinary batches: same bits as with BSI_LINEAR_ONE_CALL=0,
    sibling layers share the build, and a captured forward replays correctly after eager work in between."""
    from bsipytorch_amd import linear

    torch.manual_seed(5)
    layers = [torch.nn.Linear(512, 300).cuda(), torch.nn.Linear(512, 200, bias=False).cuda()]
    model = torch.nn.ModuleList(layers)
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    x = torch.randn(48, 512, device="cuda")
    with torch.no_grad():
        monkeypatch.setenv("BSI_LINEAR_ONE_CALL", "0")
        ref = [m(x).clone() for m in model]
        monkeypatch.setenv("BSI_LINEAR_ONE_CALL", "1")
        ops.linear_cuda_forget()
        got = [m(x).clone() for m in model]          # the second layer reuses the first one's build
        assert all(torch.equal(a, b) for a, b in zip(ref, got))
        static_x = x.clone()
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            [m(static_x) for m in model]
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        linear.forget_shared_builds()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            outs = [m(static_x) for m in model]
        linear.forget_shared_builds()
        for rep in range(3):
            static_x.copy_(x * (rep + 1))
            [m(torch.randn(20, 512, device="cuda")) for m in model]   # eager work in between overwrites the workspace
            g.replay()
            torch.cuda.synchronize()
            monkeypatch.setenv("BSI_LINEAR_ONE_CALL", "0")
            want = [m(x * (rep + 1)) for m in model]
            monkeypatch.setenv("BSI_LINEAR_ONE_CALL", "1")
            assert all(torch.equal(a, b) for a, b in zip(outs, want))


def test_few_rows_forward_captured_after_eager_runs(ops):
    """Four rows of long activations: the eager forward runs on the fused few-rows kernel, the same forward recorded
    into a graph on build + dot (the fused kernel is not free there), whose workspace must exist by then.  Replays
    give the eager bits."""
    from bsipytorch_amd import linear

    torch.manual_seed(12)
    model = torch.nn.ModuleList([torch.nn.Linear(16384, 256).cuda()])
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    layer = model[0]
    x = torch.randn(4, 16384, device="cuda")
    assert not ops.linear_few_rows_is_free(x, layer._bsi_keys_cuda)
    ops._linear_ws.clear()
    ops._reserved_linear_shapes.clear()
    with torch.no_grad():
        want = layer(x).clone()
        static_x = x.clone()
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            layer(static_x)
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        linear.forget_shared_builds()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            out = layer(static_x)
        linear.forget_shared_builds()
        for rep in range(3):
            static_x.copy_(x * (rep + 1))
            layer(torch.randn(4, 16384, device="cuda"))  # eager work in between
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, layer(x * (rep + 1)))
        assert torch.equal(want, layer(x))


def test_layer_forward_uses_the_fused_few_rows_kernel(ops, monkeypatch):
    """A decode-sized call through BSIQuantizedLinear (alone and as fused q/k/v siblings) gives the bits of the
    build + dot path, for fp32 and fp16 activations."""
    from bsipytorch_amd import linear

    class Attn(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj, self.k_proj = torch.nn.Linear(1024, 256), torch.nn.Linear(1024, 256)
            self.v_proj, self.out_proj = torch.nn.Linear(1024, 256), torch.nn.Linear(256, 1024)

        def forward(self, x):
            return self.out_proj(self.q_proj(x) + self.k_proj(x) * self.v_proj(x))

    torch.manual_seed(8)
    model = Attn().cuda()
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False, fuse_qkv=True)
    for dtype in (torch.float32, torch.float16):
        x = torch.randn(1, 3, 1024, device="cuda").to(dtype)
        monkeypatch.setenv("BSI_FUSED_LINEAR", "0")
        with torch.no_grad():
            want = model(x)
        calls = linear._sum(model, "build_calls")
        monkeypatch.setenv("BSI_FUSED_LINEAR", "1")
        with torch.no_grad():
            got = model(x)
        assert torch.equal(got, want) and got.dtype == dtype and got.shape == (1, 3, 1024)
        assert linear._sum(model, "build_calls") == calls  # no separate query build ran
