"""Pins the quantiser/packer part of the CPU oracle against independent arithmetic.

None of these checks re-types the oracle's formula: rounding is checked with exact decimal
arithmetic, the shift with ``int.bit_length``, the rounded shift with an integer closed form of
"nearest, ties away from zero", and packing by reconstructing every element from its planes.
"""
import decimal
import math

import numpy as np
import pytest


def _exact_half_away(x: float) -> int:
    """Round the exact value of the double ``x`` to the nearest integer, ties away from zero."""
    d = decimal.Decimal(x)  # exact
    r = abs(d).quantize(decimal.Decimal(1), rounding=decimal.ROUND_HALF_UP)
    return int(-r if d < 0 else r)


def test_round_half_away_grid(oracle):
    # every k + {0, .25, .5, .75} in [-300, 300]: ties must go away from zero
    for k4 in range(-1200, 1201):
        x = k4 / 4.0
        assert oracle.round_half_away(x) == _exact_half_away(x), x
    assert oracle.round_half_away(0.5) == 1
    assert oracle.round_half_away(-0.5) == -1
    assert oracle.round_half_away(2.5) == 3
    assert oracle.round_half_away(-2.5) == -3
    assert oracle.round_half_away(-0.0) == 0


def test_round_half_away_of_what_an_int64_cannot_hold(oracle):
    """The reference casts floor(x + 0.5) to long long (bsi_cuda_kernels_quant.cuh:24-29), which C++ leaves undefined
    past the int64 range; on its hardware the cast is a saturating conversion that turns a NaN into -2^63.  The oracle
    writes that out: +-(2^63 - 1) for magnitudes of 2^63 and more, infinities included; -2^63 for a NaN (it fails
    x >= 0, and the negation of -2^63 wraps); everything below 2^63 converts exactly."""
    big, small = 2 ** 63 - 1, -(2 ** 63)
    assert oracle.round_half_away(float("inf")) == big
    assert oracle.round_half_away(float("-inf")) == -big
    assert oracle.round_half_away(float("nan")) == small
    assert oracle.round_half_away(2.0 ** 63) == big and oracle.round_half_away(-(2.0 ** 63)) == -big
    assert oracle.round_half_away(1e300) == big and oracle.round_half_away(-1e300) == -big
    below = float(np.nextafter(2.0 ** 63, 0.0))  # the largest double under 2^63: an integer, converted exactly
    assert oracle.round_half_away(below) == int(below) and oracle.round_half_away(-below) == -int(below)
    # through the whole query quantiser: the chunk of such a value gets the shift of a 64-bit magnitude
    x = np.zeros((1, 512), dtype=np.float32)
    x[0, 3], x[0, 7], x[0, 300] = np.inf, 5.0, np.nan
    ints, shifts, scales = oracle.quantize_fixed(x, 2, 7, True)
    assert shifts.tolist() == [[57, 58]]           # bit_length(2^63 - 1) - 6, bit_length(2^63) - 6
    assert ints[0, 3] == 63 and ints[0, 7] == 0    # (2^63 - 1 + 2^56) >> 57 = 64, clamped to 63; 500 >> 57 = 0
    assert ints[0, 300] == -32                     # -((2^63 + 2^57) >> 58)


def test_round_to_int64_random_fp32(oracle):
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(4000).astype(np.float32),
        (rng.standard_normal(2000) * 0.02).astype(np.float32),
        (rng.integers(-5000, 5000, 2000) / 200.0).astype(np.float32),  # many values near .5 ties after *100
        np.array([0.005, -0.005, 0.015, 0.025, 1e-9, -1e-9, 655.355, -655.355, 0.0], dtype=np.float32),
    ])
    for dec in (0, 1, 2, 3):
        got = oracle.round_to_int64(x, dec)
        # (double)(float)v * 10^dec is exact for fp32 inputs and dec <= 8, and so is the + 0.5,
        # hence the result must be the exactly-rounded product.
        want = np.array([_exact_half_away(float(v) * (10.0 ** dec)) for v in x], dtype=np.int64)
        for v in x[:50]:
            assert decimal.Decimal(float(v)) * (10 ** dec) == decimal.Decimal(float(v) * (10.0 ** dec))
        np.testing.assert_array_equal(got, want)


def test_compute_shift_is_bit_length(oracle):
    for fb in (2, 6, 7, 8):
        for m in list(range(0, 5000)) + [2 ** k + o for k in range(12, 62) for o in (-1, 0, 1)]:
            want = min(62, max(0, m.bit_length() - (fb - 1)))
            assert oracle.compute_shift(m, float(m), 1, fb) == want, (m, fb)
    assert oracle.compute_shift(0, 0.0, 256, 7) == 0
    assert oracle.compute_shift(63, 0.0, 256, 7) == 0
    assert oracle.compute_shift(64, 0.0, 256, 7) == 1
    assert oracle.compute_shift(31, 0.0, 256, 6) == 0
    assert oracle.compute_shift(32, 0.0, 256, 6) == 1
    assert oracle.compute_shift(100, 0.0, 256, 0) == 0  # fixed_bits <= 0 disables


def test_compute_shift_clip(oracle):
    # clip_k caps the absmax at k * mean_abs before taking the bit width
    # max 4000, mean 10, k 8 -> effective 80 -> 7 bits -> shift 1 at fb=7
    assert oracle.compute_shift(4000, 10.0 * 256, 256, 7, 8.0) == 1
    # cap above the max leaves the max: 4000 -> 12 bits -> shift 6
    assert oracle.compute_shift(4000, 1000.0 * 256, 256, 7, 8.0) == 6
    # exact power of two boundary: effective 64 needs 7 magnitude bits
    assert oracle.compute_shift(4000, 8.0 * 256, 256, 7, 8.0) == 1
    assert oracle.compute_shift(4000, 7.99 * 256, 256, 7, 8.0) == 0


def _shift_half_away(v: int, s: int) -> int:
    # nearest integer to v / 2^s, ties away from zero, by an integer closed form
    a = abs(v)
    q = (2 * a + (1 << s)) // (1 << (s + 1))
    return -q if v < 0 else q


def test_shift_clamp_exhaustive(oracle):
    for fb in (6, 7):
        lo, hi = -(1 << (fb - 1)), (1 << (fb - 1)) - 1
        for s in range(0, 11):
            for v in range(-(1 << 12), (1 << 12) + 1, 1 if s < 4 else 3):
                want = min(hi, max(lo, _shift_half_away(v, s)))
                assert oracle.shift_clamp(v, s, fb) == want, (v, s, fb)
    # corner cases: 255 at 7 bits needs shift 2, rounds to 64, clamps to 63; -256 >> 2 == -64 is kept
    assert oracle.compute_shift(255, 0.0, 1, 7) == 2
    assert oracle.shift_clamp(255, 2, 7) == 63
    assert oracle.shift_clamp(-256, 2, 7) == -64
    assert oracle.shift_clamp(-255, 2, 7) == -64
    assert oracle.shift_clamp(3, 1, 7) == 2 and oracle.shift_clamp(-3, 1, 7) == -2  # ties away from zero
    assert oracle.shift_clamp(1, 1, 7) == 1 and oracle.shift_clamp(-1, 1, 7) == -1


@pytest.mark.parametrize("chunk", [True, False])
@pytest.mark.parametrize("fb", [6, 7])
def test_quantize_fixed_composition(oracle, chunk, fb):
    rng = np.random.default_rng(7)
    Q, d = 5, 700  # ragged: last chunk has 188 elements
    x = rng.standard_normal((Q, d)).astype(np.float32)
    x[1, 300] = 40.0   # outlier in chunk 1 only
    x[2, :256] = 0.0   # all-zero chunk
    x[3] *= 0.02
    ints, shifts, scales = oracle.quantize_fixed(x, 2, fb, chunk)
    lo, hi = -(1 << (fb - 1)), (1 << (fb - 1)) - 1
    spans = [(c * 256, min(d, c * 256 + 256)) for c in range((d + 255) // 256)] if chunk else [(0, d)]
    for q in range(Q):
        for c, (a, b) in enumerate(spans):
            r = [_exact_half_away(float(v) * 100.0) for v in x[q, a:b]]
            m = max(abs(t) for t in r)
            s = min(62, max(0, m.bit_length() - (fb - 1)))
            got_s = shifts[q, c] if chunk else shifts[q]
            got_scale = scales[q, c] if chunk else scales[q]
            assert got_s == s
            assert got_scale == float(1 << s)
            want = [min(hi, max(lo, _shift_half_away(t, s))) for t in r]
            np.testing.assert_array_equal(ints[q, a:b], np.array(want))
    if chunk:
        assert shifts[2, 0] == 0 and scales[2, 0] == 1.0      # all-zero chunk
        assert shifts[1, 1] > shifts[1, 0]                     # the outlier only moves its own chunk
    assert ints.min() >= lo and ints.max() <= hi


def test_quantize_empty_and_tail_chunk(oracle):
    x = np.ones((2, 256), dtype=np.float32)
    ints, shifts, scales = oracle.quantize_fixed(x, 2, 7, True)
    assert shifts.shape == (2, 1)
    x = np.ones((2, 257), dtype=np.float32)
    ints, shifts, scales = oracle.quantize_fixed(x, 2, 7, True)
    assert shifts.shape == (2, 2) and ints.shape == (2, 257)
    assert (shifts[:, 1] == 1).all()  # 100 needs 7 magnitude bits -> shift 1 at 7 fixed bits
    assert (ints[:, 256] == 50).all()


@pytest.mark.parametrize("S", [6, 7])
def test_pack_reconstructs(oracle, S):
    rng = np.random.default_rng(3)
    lo, hi = -(1 << (S - 1)), (1 << (S - 1)) - 1
    Q, d = 4, 333
    ints = rng.integers(lo, hi + 1, size=(Q, d)).astype(np.int64)
    ints[0, :4] = [lo, hi, 0, -1]
    words = oracle.pack(ints, S)
    W = (d + 63) // 64
    assert words.shape == (Q, S, W)
    w = oracle.slice_weights(S)  # 1, 2, 4, ..., -2^(S-1)
    assert list(w[:-1]) == [float(1 << i) for i in range(S - 1)] and w[-1] == -float(1 << (S - 1))
    rec = np.zeros((Q, W * 64), dtype=np.int64)
    for s in range(S):
        bits = ((words[:, s, :, None] >> np.arange(64, dtype=np.uint64)) & np.uint64(1)).astype(np.int64)
        rec += bits.reshape(Q, W * 64) * int(w[s])
    np.testing.assert_array_equal(rec[:, :d], ints)   # bit b of word w <-> element 64w+b
    assert (rec[:, d:] == 0).all()                     # tail bits stay zero


def test_slice_weights_unsigned_and_offset(oracle):
    assert list(oracle.slice_weights(4, 0, False)) == [1.0, 2.0, 4.0, 8.0]
    assert list(oracle.slice_weights(3, 2, True)) == [4.0, 8.0, -16.0]


def test_builders_shapes(oracle):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((3, 512)).astype(np.float32)
    qb = oracle.build_queries(x)
    assert qb["chunk_scale"] and qb["words"].shape == (3, 7, 8) and qb["scales"].shape == (3, 2)
    qb2 = oracle.build_queries(x[:, :320])  # W64 = 5 -> no chunk scales
    assert not qb2["chunk_scale"] and qb2["scales"].shape == (3,)
    kb = oracle.build_keys(x)  # sigma 1 keys: max ~ 300-400 -> 9 bits -> shift 4 at 6 fixed bits
    assert kb["words"].shape == (3, 6, 8)
    assert (kb["slice_weights"][:, 0] == kb["scales"]).all()
    assert (kb["slice_weights"][:, 5] == -32.0 * kb["scales"]).all()
    assert math.log2(kb["scales"][0]) == kb["shifts"][0] >= 3
