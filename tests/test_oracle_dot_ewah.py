"""Pins the EWAH codec and the weighted-popcount dot of the CPU oracle.

Dot: the per-chunk integer accumulator must equal the plain integer dot product of the
quantised values (numpy int64, no popcounts involved); the fp32 chain is replayed with exact
integer arithmetic and a hand-written round-to-nearest-even; the reference check scripts'
known answers are reproduced through the whole build -> dot pipeline.
EWAH: streams written by hand from the documented marker layout, round trips, size == emitted.
"""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")


def _rn_f32_int(v: int) -> int:
    """Round the integer ``v`` to the nearest value with a 24-bit significand, ties to even."""
    if v == 0:
        return 0
    s, a = (-1 if v < 0 else 1), abs(v)
    drop = a.bit_length() - 24
    if drop <= 0:
        return v
    q, rem = a >> drop, a & ((1 << drop) - 1)
    half = 1 << (drop - 1)
    if rem > half or (rem == half and (q & 1)):
        q += 1
    return s * (q << drop)


def _int_chunk_dot(a_ints, b_ints):
    """I[q,r,c] = sum over the 256-element chunk of a*b, via numpy int64 matmul."""
    Q, d = a_ints.shape
    R = b_ints.shape[0]
    chunks = (((d + 63) // 64) + 3) // 4
    out = np.zeros((Q, R, chunks), dtype=np.int64)
    for c in range(chunks):
        sl = slice(c * 256, min(d, c * 256 + 256))
        out[:, :, c] = a_ints[:, sl] @ b_ints[:, sl].T
    return out


@pytest.mark.parametrize("d", [256, 1024, 700, 64])
def test_dot_integer_identity(oracle, d):
    rng = np.random.default_rng(d)
    Q, R = 6, 9
    x = rng.standard_normal((Q, d)).astype(np.float32)
    x[0, : min(d, 256)] = np.float32(0.637) * np.sign(x[0, : min(d, 256)])  # a chunk at the clamp edge
    k = rng.standard_normal((R, d)).astype(np.float32)  # sigma 1 keys -> nonzero key shift
    k[1] *= np.float32(0.02)                             # and one row with shift 0
    qb, kb = oracle.build_queries(x), oracle.build_keys(k)
    ints, out = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    want = _int_chunk_dot(qb["ints"], kb["ints"])
    np.testing.assert_array_equal(ints.astype(np.int64), want)
    assert np.abs(want).max() <= 256 * 64 * 32


def test_dot_extreme_values_no_overflow(oracle):
    # all queries -64, all keys -32: I = 256*64*32 = 2^19 per chunk, the largest magnitude possible
    Q, R, d = 2, 3, 512
    a = np.full((Q, d), -64, dtype=np.int64)
    b = np.full((R, d), -32, dtype=np.int64)
    b[1] = 31
    a[1] = 63
    A, B = oracle.pack(a, 7), oracle.pack(b, 6)
    ints, _ = oracle.dot_fixed(A, np.ones((Q, 2), np.float32), B, np.ones(R, np.float32), 1.0)
    np.testing.assert_array_equal(ints.astype(np.int64), _int_chunk_dot(a, b))
    assert ints[0, 0, 0] == 1 << 19


def test_dot_fp32_chain_exact_replay(oracle):
    rng = np.random.default_rng(11)
    Q, R, d = 4, 5, 256 * 40  # 40 chunks so that the fp32 accumulator does round
    a = rng.integers(40, 64, size=(Q, d)).astype(np.int64)        # same-sign, large: partial sums pass 2^24
    b = rng.integers(20, 32, size=(R, d)).astype(np.int64)
    a[1] = -a[1]
    A, B = oracle.pack(a, 7), oracle.pack(b, 6)
    qscale = (2.0 ** rng.integers(0, 8, size=(Q, 40))).astype(np.float32)
    bscale = (2.0 ** rng.integers(0, 5, size=R)).astype(np.float32)
    sinv = oracle.scale_inv(2, 2)
    ints, out = oracle.dot_fixed(A, qscale, B, bscale, sinv)
    rounded_somewhere = False
    for q in range(Q):
        for r in range(R):
            acc = 0
            for c in range(40):
                exact = acc + int(ints[q, r, c]) * int(qscale[q, c]) * int(bscale[r])  # fma: one rounding
                acc = _rn_f32_int(exact)
                rounded_somewhere |= (acc != exact)
            # acc * scale_inv: the product of two fp32 values is exact in fp64, so one rounding to fp32
            want = np.float32(np.float64(acc) * np.float64(sinv))
            assert out[q, r] == want, (q, r)
    assert rounded_somewhere, "test too weak: the fp32 accumulator never rounded"
    assert sinv == np.float32(1e-4)


@pytest.mark.parametrize("bits_q,bits_k", [(33, 20), (16, 16), (40, 23), (2, 63), (63, 63)])
def test_dot_wide_operands_against_python_integers(oracle, bits_q, bits_k):
    """Widths up to the 63 bits the reference's flags allow: the chunk integer is the exact dot while it fits 64 bits
    (Python integers, no popcounts), its low 32 bits are what the int32 output holds, and float(I) enters the chain
    with one rounding.  With 63 x 63 bits the dot does not fit: then the oracle's integer is the dot modulo 2^64."""
    rng = np.random.default_rng(bits_q * 64 + bits_k)
    Q, R, d = 3, 4, 512
    a = rng.integers(-(1 << (bits_q - 1)), 1 << (bits_q - 1), size=(Q, d), dtype=np.int64)
    b = rng.integers(-(1 << (bits_k - 1)), 1 << (bits_k - 1), size=(R, d), dtype=np.int64)
    a[0, :256] = -(1 << (bits_q - 1))  # a chunk of the most negative value on both sides
    b[0, :256] = -(1 << (bits_k - 1))
    A, B = oracle.pack(a, bits_q), oracle.pack(b, bits_k)
    ints, out = oracle.dot_fixed(A, np.ones((Q, 2), np.float32), B, np.ones(R, np.float32), 1.0)
    for q in range(Q):
        for r in range(R):
            acc = 0
            for c in range(2):
                exact = sum(int(x) * int(y) for x, y in zip(a[q, c * 256:(c + 1) * 256], b[r, c * 256:(c + 1) * 256]))
                if bits_q + bits_k + 8 <= 63:
                    assert abs(exact) < 1 << 63
                wrapped = (exact + (1 << 63)) % (1 << 64) - (1 << 63)  # the signed 64-bit reading of exact mod 2^64
                low = wrapped & 0xFFFFFFFF
                assert int(ints[q, r, c]) == (low - (1 << 32) if low >> 31 else low), (q, r, c)
                # fmaf(float(I), 1, acc): float(I) rounds once, the exact sum of the two fp32 values once more
                acc = _rn_f32_int(acc + _rn_f32_int(wrapped))
            assert out[q, r] == np.float32(acc), (q, r)


def test_dot_row_scale_and_partial_chunk(oracle):
    # W64 = 5: no chunk scales (one scale per row), last chunk holds a single word
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, 320)).astype(np.float32)
    k = (rng.standard_normal((4, 320)) * 0.02).astype(np.float32)
    qb, kb = oracle.build_queries(x), oracle.build_keys(k)
    assert not qb["chunk_scale"]
    ints, out = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    assert ints.shape == (3, 4, 2)
    np.testing.assert_array_equal(ints.astype(np.int64), _int_chunk_dot(qb["ints"], kb["ints"]))
    deq = (qb["ints"] * qb["scales"][:, None]) @ (kb["ints"] * kb["scales"][:, None]).T / 1e4
    np.testing.assert_allclose(out, deq, rtol=1e-6)


def test_reference_known_answers(oracle):
    kat = json.load(open(GOLDEN))
    for case in kat["vector_dot"]:
        q = np.array([case["q"]], dtype=np.float32)
        k = np.array([case["k"]], dtype=np.float32)
        dec = case["decimal_places"]
        qb, kb = oracle.build_queries(q, dec), oracle.build_keys(k, dec, case["key_bits"])
        assert (qb["shifts"] == 0).all() and (kb["shifts"] == 0).all()
        _, out = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(dec, dec))
        assert abs(float(out[0, 0]) - case["expected"]) < 0.01, case["cite"]   # the reference scripts' tolerance
        assert float(out[0, 0]) == np.float32(case["expected"]), case["cite"]  # and in fact exact
    for case in kat["batch_dot"]:
        q = np.array(case["q"], dtype=np.float32)
        K = np.array(case["K"], dtype=np.float32)
        dec = case["decimal_places"]
        qb, kb = oracle.build_queries(q, dec), oracle.build_keys(K, dec, case["key_bits"])
        _, out = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(dec, dec))
        np.testing.assert_array_equal(out, np.array(case["expected"], dtype=np.float32), err_msg=case["cite"])


def test_accuracy_vs_dense_matmul(oracle):
    # statistical bound, not allclose: keys ~N(0, 0.02) sit on a 0.01 grid after decimal_places=2
    rng = np.random.default_rng(123)
    x = rng.standard_normal((16, 2048)).astype(np.float32)
    k = (rng.standard_normal((32, 2048)) * 0.02).astype(np.float32)
    qb, kb = oracle.build_queries(x), oracle.build_keys(k)
    _, out = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    dense = x.astype(np.float64) @ k.astype(np.float64).T
    rel = np.linalg.norm(out - dense) / np.linalg.norm(dense)
    cos = (out * dense).sum() / (np.linalg.norm(out) * np.linalg.norm(dense))
    assert rel < 0.25 and cos > 0.97, (rel, cos)


# ---------------- EWAH ----------------

ONES = np.uint64(0xFFFFFFFFFFFFFFFF)


def _marker(run_bit, run_len, lit):
    return np.uint64(run_bit | (run_len << 1) | (lit << 33))


def test_ewah_flags_thresholds(oracle):
    W = 128  # 8192 bits
    def with_bits(n):
        w = np.zeros(W, dtype=np.uint64)
        for b in range(n):
            w[b % W] |= np.uint64(1) << np.uint64(b // W)
        return w
    words = np.stack([with_bits(0), with_bits(8192), with_bits(40), with_bits(48), with_bits(4096), with_bits(8192 - 40)])
    flags = oracle.compress_flags(words, 0.5)
    # p = 0 and p = 1 give M = 0; 1-(1-p)^128 crosses 0.5 at p = 0.0054 (between 40 and 48 set bits of 8192)
    assert list(flags) == [1, 1, 1, 0, 0, 1]
    assert list(oracle.compress_flags(words, 0.0)) == [1, 1, 0, 0, 0, 0]
    assert list(oracle.compress_flags(words, 1.0)) == [1, 1, 1, 1, 1, 1]


def test_ewah_hand_built_streams(oracle):
    lit1, lit2 = np.uint64(0x00F0), np.uint64(0x8000000000000001)
    words = np.array([[0, 0, 0, lit1, lit2, ONES, ONES, 0]], dtype=np.uint64)
    stream, off, lens = oracle.ewah_encode(words, np.array([1], dtype=np.int32))
    want = [_marker(0, 3, 2), lit1, lit2, _marker(1, 2, 0), _marker(0, 1, 0)]
    assert list(stream) == want and lens[0] == 5 and off[0] == 0
    np.testing.assert_array_equal(oracle.ewah_decompress(stream, 8), words[0])
    # flag 0: a single marker with lit_count = W, then W literals (even if they are clean words)
    stream, _, lens = oracle.ewah_encode(words, np.array([0], dtype=np.int32))
    assert lens[0] == 9 and stream[0] == _marker(0, 0, 8)
    np.testing.assert_array_equal(stream[1:], words[0])
    # all-zero slice: one marker, run_len = W
    z = np.zeros((1, 32), dtype=np.uint64)
    stream, _, lens = oracle.ewah_encode(z, np.array([1], dtype=np.int32))
    assert list(stream) == [_marker(0, 32, 0)]
    # decode pads with zeros when the stream is short and stops at W when it is long
    np.testing.assert_array_equal(oracle.ewah_decompress(np.array([_marker(1, 2, 0)], dtype=np.uint64), 4),
                                  np.array([ONES, ONES, 0, 0], dtype=np.uint64))
    np.testing.assert_array_equal(oracle.ewah_decompress(np.array([_marker(1, 9, 0)], dtype=np.uint64), 4),
                                  np.array([ONES] * 4, dtype=np.uint64))
    np.testing.assert_array_equal(oracle.ewah_decompress(np.zeros(0, dtype=np.uint64), 3), np.zeros(3, dtype=np.uint64))


@pytest.mark.parametrize("seed", range(6))
def test_ewah_round_trip(oracle, seed):
    rng = np.random.default_rng(seed)
    S, W = 7, 64 + seed
    words = rng.integers(0, 2 ** 63, size=(S, W)).astype(np.uint64)
    words[0] = 0
    words[1] = ONES
    words[2, rng.random(W) < 0.7] = 0
    words[3, rng.random(W) < 0.7] = ONES
    words[4, 10:40] = 0
    words[4, 40:50] = ONES
    for flags in (np.ones(S, np.int32), np.zeros(S, np.int32), oracle.compress_flags(words, 0.5)):
        stream, off, lens = oracle.ewah_encode(words, flags)
        assert off[0] == 0 and (np.diff(off) == lens[:-1]).all() and lens.sum() == stream.size
        for s in range(S):
            np.testing.assert_array_equal(oracle.ewah_decompress(stream[off[s]: off[s] + lens[s]], W), words[s])
            if not flags[s]:
                assert lens[s] == W + 1
        if flags[0]:
            assert lens[0] == 1 and lens[1] == 1


def _drawn_planes(rng, S, W):
    """Slices made of stretches of zeros, ones, random literals and one-bit literals of drawn lengths."""
    words = np.zeros((S, W), dtype=np.uint64)
    for s in range(S):
        w = 0
        while w < W:
            n = min(int(rng.choice([1, 1, 2, 3, 7, 63, 64, 65, 130])), W - w)
            kind = rng.integers(0, 4)
            if kind == 1:
                words[s, w:w + n] = ONES
            elif kind == 2:
                words[s, w:w + n] = rng.integers(1, 2 ** 63, size=n, dtype=np.uint64) * np.uint64(2)
            elif kind == 3:
                words[s, w:w + n] = np.uint64(1) << rng.integers(0, 64, size=n, dtype=np.uint64)
            w += n
    return words


@pytest.mark.parametrize("seed", range(12))
def test_ewah_stream_length_and_fields_in_closed_form(oracle, seed):
    """What the greedy encoder must produce, stated without walking the slice: a marker for every maximal run of equal
    clean words plus one if the slice starts with a literal, and every literal once -- so the stream length is a count
    over the words; the markers' run lengths and literal counts add up to W; the runs name the clean words' kind and the
    payload is the literal words in order.  (A dropped marker, a run split in two, a literal counted with the wrong
    marker or a field one bit off fails one of these.)"""
    rng = np.random.default_rng(100 + seed)
    S, W = 9, int(rng.choice([1, 5, 64, 65, 200, 513]))
    words = _drawn_planes(rng, S, W)
    stream, off, lens = oracle.ewah_encode(words, np.ones(S, dtype=np.int32))
    for s in range(S):
        row = words[s]
        clean = (row == 0) | (row == ONES)
        prev_same = np.zeros(W, dtype=bool)
        prev_same[1:] = clean[1:] & clean[:-1] & (row[1:] == row[:-1])
        run_starts = int((clean & ~prev_same).sum())
        want_len = int((~clean).sum()) + run_starts + (0 if clean[0] else 1)
        assert lens[s] == want_len
        st = stream[off[s]: off[s] + lens[s]]
        i, covered, payload = 0, 0, []
        while i < len(st):
            m = int(st[i])
            run_bit, run_len, lit = m & 1, (m >> 1) & 0xFFFFFFFF, m >> 33
            if run_len:
                assert (row[covered: covered + run_len] == (ONES if run_bit else 0)).all()
            else:
                assert run_bit == 0 and covered == 0  # only a slice that starts with a literal has a marker without a run
            covered += run_len
            payload.extend(st[i + 1: i + 1 + lit])
            assert not clean[covered: covered + lit].any()
            covered += lit
            i += 1 + lit
        assert covered == W and i == len(st)
        np.testing.assert_array_equal(np.array(payload, dtype=np.uint64), row[~clean])


def test_relu_queries_sign_plane_is_one_run(oracle):
    # ReLU'd activations: the sign plane is all zero -> a single run marker; dense planes stay verbatim
    rng = np.random.default_rng(9)
    x = np.maximum(rng.standard_normal((1, 8192)), 0).astype(np.float32)
    qb = oracle.build_queries(x)
    planes = qb["words"][0]
    flags = oracle.compress_flags(planes, 0.5)
    assert flags[6] == 1 and flags[0] == 0
    stream, off, lens = oracle.ewah_encode(planes, flags)
    assert lens[6] == 1 and stream[off[6]] == _marker(0, 128, 0)
    assert lens[0] == 129
