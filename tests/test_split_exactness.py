"""The arithmetic fact the D-split launches of the int8-image dot rest on, checked on the CPU with exact integers.

The chunk chain of the reference (bsi_cuda_kernels_dot.cuh:1516-1540) is acc = fmaf(float(I_c), scale_c, acc) over the
chunks in order, with integer I_c and power-of-two scales: every operand is an integer times one power of two, so the
chain can be replayed exactly in Python integers with a correctly rounded float32 step.  The kernel's claim: run the
chain over `segments` runs of chunks, each from zero, and follow the largest magnitude each run's values take; if every
run's peak is at most 2^24 units / segments (rounded down to a power of two), then the sum of the runs' results, in any
order, IS the sequential chain's result -- and a run over the limit says nothing, which is why the kernel then computes
the tile again in order.  `unit` is the kernel's 2^(16 - Sa - Sb) (its accumulators carry that multiple of I_c)."""
import itertools
import random

import pytest


def fl32(v: int) -> int:
    """Round an integer to the nearest integer a float32 holds (24-bit significand, ties to even): what one fmaf
    step does to acc + I * scale when all of them are integers and nothing overflows."""
    a = abs(v)
    if a < (1 << 24):
        return v
    shift = a.bit_length() - 24
    q, r = a >> shift, a & ((1 << shift) - 1)
    half = 1 << (shift - 1)
    if r > half or (r == half and (q & 1)):
        q += 1
    return (q << shift) if v >= 0 else -(q << shift)


def chain(terms):
    """(final value, peak magnitude) of the fp32 chain over integer terms, from zero."""
    acc, peak = 0, 0
    for t in terms:
        acc = fl32(acc + t)
        peak = max(peak, abs(acc))
    return acc, peak


def split_runs(n, segments):
    """The kernel's runs of chunks: segment s takes chunks [n s / segments, n (s + 1) / segments)."""
    return [(n * s // segments, n * (s + 1) // segments) for s in range(segments)]


def limit(unit_log2, segments):
    return 1 << (24 + unit_log2 - (segments - 1).bit_length())


def test_fl32_is_round_to_nearest_even():
    import numpy as np

    rng = random.Random(1)
    for _ in range(20000):
        v = rng.randrange(-(1 << 40), 1 << 40)
        assert fl32(v) == int(np.float32(v))
    for v in ((1 << 24) + 1, (1 << 24) + 3, (1 << 25) + 2, (1 << 25) + 6, -((1 << 24) + 1)):
        assert fl32(v) == int(np.float32(v))   # ties


@pytest.mark.parametrize("seed", range(8))
def test_runs_within_the_limit_add_up_to_the_sequential_chain(seed):
    rng = random.Random(seed)
    checked = 0
    for _ in range(3000):
        n = rng.randrange(2, 65)
        segments = rng.randrange(2, min(n, 16) + 1)
        unit_log2 = rng.choice([0, 3, 7])
        big = rng.random() < 0.5
        # terms = unit * I_c * 2^shift_c; magnitudes drawn so that about half the cases sit near the limit
        mag = rng.choice([12, 16, 19]) if big else rng.choice([4, 8, 12])
        terms = [(rng.randrange(-(1 << mag), (1 << mag) + 1) << rng.randrange(0, 8 if big else 4)) << unit_log2 for _ in range(n)]
        if rng.random() < 0.3:
            terms = [abs(t) for t in terms]            # same sign: prefixes grow fastest
        runs = [chain(terms[a:b]) for a, b in split_runs(n, segments)]
        lim = limit(unit_log2, segments)
        if all(peak <= lim for _, peak in runs):
            sequential, _ = chain(terms)
            parts = [v for v, _ in runs]
            assert sum(parts) == sequential == sum(terms)       # exact, hence the same in any order of addition
            rng.shuffle(parts)
            acc = 0
            for p in parts:                                     # the last workgroup's float additions, any order
                acc = fl32(acc + p)
            assert acc == sequential
            checked += 1
    assert checked > 300   # the draw does reach the claim's side often enough


def test_the_limit_is_tight_enough_to_matter_and_a_run_over_it_can_differ():
    # at the limit exactly: still exact
    for segments, unit_log2 in itertools.product((2, 3, 4, 8), (0, 3)):
        lim = limit(unit_log2, segments)
        terms = [lim] * segments                       # one chunk per run, each at the limit
        runs = [chain(terms[a:b]) for a, b in split_runs(len(terms), segments)]
        assert all(peak == lim for _, peak in runs)
        assert sum(v for v, _ in runs) == chain(terms)[0]
    # beyond it the sequential chain rounds, and the runs' sum is not its value: the kernel must recompute in order
    terms = [(1 << 24) + 1, 1, 1, 1]
    sequential, _ = chain(terms)
    runs = [chain(terms[a:b]) for a, b in split_runs(4, 2)]
    assert any(peak > limit(0, 2) for _, peak in runs)
    assert sum(v for v, _ in runs) != sequential
