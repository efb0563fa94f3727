"""Pins the oracle's restatement of the reference's scalar entry points (values only).

Independent checks: the known answers of the reference's own check scripts, hand-worked truncation and rounding
cases, and exact rational arithmetic (fractions) on small inputs.
"""
import json
import os
from fractions import Fraction

import numpy as np

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")


def test_trunc_scaled_hand_worked(oracle):
    x = np.array([0.999, -0.999, 2.5, -2.5, 1e-3, 3.0, -0.0], dtype=np.float32)
    assert oracle.trunc_scaled(x, 10.0).tolist() == [9, -9, 25, -25, 0, 30, 0]          # towards zero, not to nearest
    assert oracle.trunc_scaled(x, 1000.9).tolist() == [999, -999, 2500, -2500, 1, 3000, 0]  # the factor is cast to long first
    # the product is formed in float: 16777217 is not a float, 16777216 * 1 stays, 0.1f * 10 rounds to 1.0f exactly
    assert oracle.trunc_scaled(np.array([0.1], dtype=np.float32), 10.0).tolist() == [1]
    assert oracle.trunc_scaled(np.array([0.7], dtype=np.float32), 10.0).tolist() == [6 if np.float32(0.7) * np.float32(10) < 7 else 7]


def test_scalar_dots_reproduce_the_reference_scripts_answers(oracle):
    g = json.load(open(GOLDEN))
    for case in g["vector_dot"]:
        q, k = np.array(case["q"], dtype=np.float32), np.array(case["k"], dtype=np.float32)
        for dec in (case["decimal_places"], 2, 4):
            assert oracle.scalar_dot_product_decimal(q, k, dec) == case["expected"], case["cite"]
        assert abs(oracle.scalar_dot_product(q, k, 1000.0) - case["expected"]) < 0.01, case["cite"]
    for case in g["batch_dot"]:
        K = np.array(case["K"], dtype=np.float32)
        for qi, qrow in enumerate(case["q"]):
            out = oracle.scalar_batch_dot_product(np.array(qrow, dtype=np.float32), K, case["decimal_places"])
            assert out.tolist() == [float(v) for v in case["expected"][qi]], case["cite"]


def test_scalar_dots_against_exact_rationals(oracle):
    rng = np.random.default_rng(3)
    m = (rng.integers(-999, 999, size=50) / 100.0).astype(np.float32)   # two decimals: x * 100 rounds to the integer
    n = (rng.integers(-999, 999, size=50) / 100.0).astype(np.float32)
    mi = [round(Fraction(float(v)) * 100) for v in m]
    ni = [round(Fraction(float(v)) * 100) for v in n]
    exact = sum(a * b for a, b in zip(mi, ni))
    assert oracle.scalar_dot_product_decimal(m, n, 2) == exact / 10000.0
    # one decimal place less: ties such as 0.25 * 10 = 2.5 go away from zero
    t = np.array([0.25, -0.25, 0.35], dtype=np.float32)
    # 0.35f is 0.3499999940...: times 10 in double it stays below 3.5 and rounds to 3; the ones round to 10
    assert float(np.float32(0.35)) * 10 < 3.5
    assert oracle.scalar_dot_product_decimal(t, np.ones(3, dtype=np.float32), 1) == (3 - 3 + 3) * 10 / 100.0


def test_vector_dot_product_wraps_to_32_bits(oracle):
    m = np.full(8, 30000.0, dtype=np.float32)
    n = np.full(8, 30000.0, dtype=np.float32)
    # 8 * 9e8 = 7.2e9 does not fit an int: the reference's accumulator keeps the low 32 bits
    assert oracle.scalar_vector_dot_product(m, n, 1.0) == (7200000000 + 2**31) % 2**32 - 2**31
    assert oracle.scalar_vector_dot_product(np.array([1.5, 2.0], dtype=np.float32), np.array([2.0, 3.0], dtype=np.float32), 10.0) == 15 * 20 + 20 * 30
