"""The reference's scalar bsi_ops entry points (bsiFunctions.cpp:811-846), served by the device kernels.

Values are checked against what the reference's own source fixes -- its stated integer rule, an exact integer dot
computed independently in numpy, the stated divisor -- and against the known answers its check scripts hold.
Byte counts and slice statistics describe this build's slices (the bsiCPP containers are not in the reference's
tree): they are checked for consistency only, parity unpinned.
"""
import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")


@pytest.fixture(scope="module")
def ops():
    import bsi_ops

    return bsi_ops


def _round_half_away(x, dec):
    v = x.astype(np.float64) * 10.0 ** dec
    return np.where(v >= 0, np.floor(v + 0.5), -np.floor(-v + 0.5)).astype(np.int64)


def test_known_answers_of_the_reference_scripts(ops):
    g = json.load(open(GOLDEN))
    for case in g["vector_dot"]:
        q, k = torch.tensor(case["q"], dtype=torch.float32), torch.tensor(case["k"], dtype=torch.float32)
        for dec in (case["decimal_places"], 2, 3):
            res, ns, b1, b2 = ops.dot_product_decimal(q, k, dec)
            assert abs(res - case["expected"]) < 1e-9, case["cite"]
            assert ns >= 0 and b1 > 0 and b2 > 0
        # test.py:9-12 and test_bsi_simple.py call dot_product with a precision factor
        res, _, _, _ = ops.dot_product(q, k, 1000.0)
        assert abs(res - case["expected"]) < 0.01, case["cite"]
    for case in g["batch_dot"]:
        K = torch.tensor(case["K"], dtype=torch.float32)
        for qi, qrow in enumerate(case["q"]):
            q = torch.tensor(qrow, dtype=torch.float32)
            out, ns, mq, mk = ops.batch_dot_product(q, K, case["decimal_places"])
            assert out.dtype == torch.float64 and out.device.type == "cpu"
            np.testing.assert_array_equal(out.numpy(), np.array(case["expected"][qi], dtype=np.float64), err_msg=case["cite"])
            cap, total, num_keys, d = ops.build_bsi_keys(K, 2, 0.2)
            assert (num_keys, d) == tuple(K.shape) and total > 0
            out2, total_ns, build_ns, dot_ns, mem_q = ops.batch_dot_product_prebuilt(q, cap)
            np.testing.assert_array_equal(out2.numpy(), np.array(case["expected"][qi], dtype=np.float64))
            assert total_ns == build_ns + dot_ns
            qcap, qbytes, slices = ops.build_bsi_query(q, 2)
            out3, t3, zero, d3, mq3 = ops.batch_dot_product_prebuilt_capsule(qcap, cap)
            np.testing.assert_array_equal(out3.numpy(), out2.numpy())
            assert zero == 0 and t3 == d3 and mq3 == qbytes and slices >= 2


@pytest.mark.parametrize("n,dec", [(1, 2), (63, 0), (64, 1), (1000, 2), (4097, 3)])
def test_dot_product_decimal_is_the_exact_integer_dot(ops, oracle, n, dec):
    rng = np.random.default_rng(n + dec)
    m = (rng.standard_normal(n) * 7).astype(np.float32)
    k = (rng.standard_normal(n) * 0.3).astype(np.float32)
    res, _, _, _ = ops.dot_product_decimal(torch.from_numpy(m), torch.from_numpy(k).cuda(), dec)
    exact = int(_round_half_away(m, dec) @ _round_half_away(k, dec))
    assert res == exact / (10.0 ** (2 * dec) if dec > 0 else 1.0)
    assert res == oracle.scalar_dot_product_decimal(m, k, dec)


@pytest.mark.parametrize("pf", [1.0, 10.0, 1000.0, 12345.0])
def test_dot_product_truncates_the_float_product(ops, oracle, pf):
    rng = np.random.default_rng(int(pf))
    m = (rng.standard_normal(777) * 3).astype(np.float32)
    k = (rng.standard_normal(777) * 3).astype(np.float32)
    m[:4] = [0.999, -0.999, 2.0005, -1e-3]
    factor = np.float32(int(pf))
    im, ik = (m * factor).astype(np.int64), (k * factor).astype(np.int64)   # float32 product, towards zero
    res, _, _, _ = ops.dot_product(torch.from_numpy(m), torch.from_numpy(k), pf)
    assert res == float(int(im @ ik)) / float(np.float32(np.float32(pf) * np.float32(pf)))
    assert res == oracle.scalar_dot_product(m, k, pf)
    # the plain-integer baselines: same integers, int accumulator (32 bits), no division
    v, _, b1, b2, bits1, bits2 = ops.vector_dot_product(torch.from_numpy(m), torch.from_numpy(k), pf)
    want = (int(im @ ik) + (1 << 31)) % (1 << 32) - (1 << 31)
    assert v == want and (b1, b2, bits1, bits2) == (1024 * 8, 1024 * 8, 64, 64)
    assert v == oracle.scalar_vector_dot_product(m, k, pf)


def test_random_number_and_int16_variants(ops):
    rng = np.random.default_rng(5)
    m = (rng.standard_normal(300) * 100).astype(np.float32)
    k = (rng.standard_normal(300) * 100).astype(np.float32)
    want = int(m.astype(np.int64) @ k.astype(np.int64))
    r1, _ = ops.random_number_dot_product_bsi(torch.from_numpy(m), torch.from_numpy(k))
    r2, _ = ops.random_number_dot_product_vector(torch.from_numpy(m), torch.from_numpy(k))
    r3, _, b1, b2, bits1, bits2 = ops.vector_dot_product_no_precison(torch.from_numpy(m), torch.from_numpy(k))
    assert r1 == float(want) and r2 == want and r3 == want
    assert (b1, b2, bits1, bits2) == (600, 600, 16, 16)


def test_batch_against_integer_matrix_product_and_capsules(ops, oracle, tmp_path):
    rng = np.random.default_rng(9)
    K = (rng.standard_normal((37, 300)) * 0.5).astype(np.float32)
    K[3] = np.abs(K[3])
    K[5] = 0.0
    q = rng.standard_normal(300).astype(np.float32)
    dec = 2
    want = (_round_half_away(K, dec) @ _round_half_away(q, dec)).astype(np.float64) / 10.0 ** (2 * dec)
    out, _, mem_q, mem_k0 = ops.batch_dot_product(torch.from_numpy(q), torch.from_numpy(K), dec)
    np.testing.assert_array_equal(out.numpy(), want)
    np.testing.assert_array_equal(out.numpy(), oracle.scalar_batch_dot_product(q, K, dec))
    cap, total, R, d = ops.build_bsi_keys(torch.from_numpy(K), dec, 0.5)
    out2, _, _, _, mem_q2 = ops.batch_dot_product_prebuilt(torch.from_numpy(q), cap, 0.5)
    np.testing.assert_array_equal(out2.numpy(), want)
    assert mem_q > 0 and mem_k0 > 0 and mem_q2 > 0
    # statistics are consistent with each other
    st = ops.keyset_slice_stats(cap)
    assert st["num_vectors"] == 37 and st["total_slices"] == st["verbatim_slices"] + st["compressed_slices"]
    assert st["total_slices"] % 37 == 0 and abs(st["compressed_pct"] + st["verbatim_pct"] - 100.0) < 1e-9
    assert st["compressed_slices"] > 0      # row 5 is all zero: its slices compress
    ts = ops.tensor_slice_stats(torch.from_numpy(K[5]), dec, 0.5)
    assert ts["verbatim_slices"] == 0 and ts["total_slices"] == 2 and ts["memory_bytes"] == 2 * 8 and ts["signed_input"]
    mem, disk = ops.keyset_size_on_disk(cap)
    assert mem == total and disk > 0
    ops.save_keyset(cap, str(tmp_path / "ks"))
    assert os.path.getsize(tmp_path / "ks" / "keyset.bsik") == disk
    loaded, _, R2, d2, _ = ops.load_keyset_cuda(str(tmp_path / "ks"))
    assert (R2, d2) == (37, 300)
    # the saved planes stand for the same integers: decimal queries against them give the same scores
    os.environ["BSI_FIXED_BITS_QUERIES"] = "0"
    ops._reset_flag_cache()
    try:
        qcap = ops.build_bsi_queries_cuda_batch_packed(torch.from_numpy(q).unsqueeze(0).cuda(), dec, 0.5)
        scores = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, loaded)[0]
    finally:
        del os.environ["BSI_FIXED_BITS_QUERIES"]
        ops._reset_flag_cache()
    np.testing.assert_allclose(scores.cpu().numpy()[0], want, rtol=1e-6, atol=0)  # fp32 scale there, float64 division here
    # query words: two's-complement planes of the rounded integers, least significant slice first
    qc, qbytes, S = ops.build_bsi_query(torch.from_numpy(q), dec)
    words, rows, offset, decimals, twos = ops.debug_bsi_query_words(qc)
    assert rows == 300 and offset == 0 and decimals == dec and twos and tuple(words.shape) == (S, 5)
    ints = _round_half_away(q, dec)
    e = np.arange(300)
    bits = (words.numpy().view(np.uint64)[:, e >> 6] >> (e & 63).astype(np.uint64)) & np.uint64(1)
    weights = np.array([1 << s for s in range(S - 1)] + [-(1 << (S - 1))], dtype=np.int64)
    np.testing.assert_array_equal((bits.astype(np.int64) * weights[:, None]).sum(axis=0), ints)


def test_argument_checks(ops):
    with pytest.raises(RuntimeError, match="q.size\\(0\\) must equal K.size\\(1\\)"):
        ops.batch_dot_product(torch.zeros(3), torch.zeros(2, 4), 2)
    with pytest.raises(RuntimeError, match="must be 1D"):
        ops.dot_product(torch.zeros(2, 2), torch.zeros(2), 10.0)
    cap, _, _, _ = ops.build_bsi_keys(torch.ones(2, 4), 1)
    with pytest.raises(RuntimeError, match="keys' dimension"):
        ops.batch_dot_product_prebuilt(torch.zeros(3), cap)
    with pytest.raises(RuntimeError, match="Invalid BSI query capsule"):
        ops.batch_dot_product_prebuilt_capsule(cap, cap)
    # empty inputs
    res, _, _, _ = ops.dot_product_decimal(torch.zeros(0), torch.zeros(0), 2)
    assert res == 0.0
