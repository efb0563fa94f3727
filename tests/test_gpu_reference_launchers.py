"""The reference's own launcher symbols (libbsi_reference_launchers.so), called through ctypes with the reference's
exact argument lists and in the order its C++ calls them, against the oracle:

  keys     bsi_cuda_quantize_to_int64_and_scale (bsi_vector_cuda.cpp:581-656): launch_quantize_round_to_int64_batch,
           launch_compute_row_shift_scale, launch_apply_row_shift_clamp; then launch_pack_bits_all_ballot_batch (:1125)
  queries  bsi_cuda_build_fixed_query_words_fused (:401-557): launch_compute_chunk_shift_scale_from_input,
           launch_quantize_shift_pack_chunk_batch
  dot      batch_dot_product_multiquery_cuda_batch_caps (bsi_cuda.cpp:724-746):
           launch_popcount_weighted_keys_literal_fused_multiq, 19 arguments
  codec    launch_slice_popcount_sum, launch_compress_flags_from_density, launch_ewah_size, launch_ewah_emit,
           launch_ewah_decompress (bsi_vector_cuda.cpp:896-951, bsi_cuda.cpp:402-414)
"""
import ctypes
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
vp, i32, i64, f32, f64, u64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_double, ctypes.c_uint64


@pytest.fixture(scope="module")
def launchers():
    L = ctypes.CDLL(os.path.join(ROOT, "bsipytorch_amd", "libbsi_reference_launchers.so"))
    sig = {
        "launch_quantize_round_to_int64_batch": [vp, i32, i64, i64, f64, vp, vp],
        "launch_compute_row_shift_scale": [vp, i64, i64, i32, f32, vp, vp, vp],
        "launch_apply_row_shift_clamp": [vp, i64, i64, vp, i32, vp],
        "launch_pack_bits_all_ballot_batch": [vp, i32, ctypes.c_longlong, i32, i32, u64, vp, vp],
        "launch_compute_chunk_shift_scale_from_input": [vp, i32, i64, i64, i32, f64, i32, f32, vp, vp, vp],
        "launch_quantize_shift_pack_chunk_batch": [vp, i32, i64, i64, i32, i32, i32, u64, f64, i32, vp, vp, vp],
        "launch_popcount_weighted_keys_literal_fused_multiq": [vp, vp, vp, i32, i32, i32, vp, vp, i32, i32, i32, i32, i32,
                                                               vp, vp, f32, i32, vp, vp],
        "launch_slice_popcount_sum": [vp, i32, i32, vp, vp],
        "launch_compress_flags_from_density": [vp, i32, i32, f64, vp, vp],
        "launch_ewah_size": [vp, i32, i32, vp, vp, vp],
        "launch_ewah_emit": [vp, i32, i32, vp, vp, vp, vp, vp],
        "launch_ewah_decompress": [vp, i32, i32, vp, vp],
    }
    for name, args in sig.items():
        fn = getattr(L, name)
        fn.argtypes, fn.restype = args, None
    L.bsi_launchers_last_error.restype = ctypes.c_char_p
    return L


def _ok(L):
    assert L.bsi_launchers_last_status() == 0, L.bsi_launchers_last_error()


def _st():
    return torch.cuda.current_stream().cuda_stream


@pytest.mark.parametrize("Q,R,d", [(64, 256, 2048), (130, 75, 1024), (600, 40, 16384)])
def test_reference_call_sequence_through_the_launchers(launchers, oracle, Q, R, d):
    L = launchers
    L.bsi_launchers_clear_status()
    rng = np.random.default_rng(Q + R)
    x = rng.standard_normal((Q, d)).astype(np.float32)
    x[:, rng.permutation(d)[:2]] *= 20.0
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    k[1] *= 60.0
    W, chunks = d // 64, d // 256
    st = _st()
    # keys: round, row shift/scale, shift + clamp, pack 6 planes; slice weights as bsi_vector_cuda.cpp:1144-1158
    kd = torch.from_numpy(k).cuda()
    kints = torch.empty((R, d), dtype=torch.int64, device="cuda")
    kshift = torch.empty((R,), dtype=torch.int32, device="cuda")
    kscale = torch.empty((R,), dtype=torch.float32, device="cuda")
    L.launch_quantize_round_to_int64_batch(kd.data_ptr(), 0, R, d, 100.0, kints.data_ptr(), st)
    L.launch_compute_row_shift_scale(kints.data_ptr(), R, d, 6, 0.0, kshift.data_ptr(), kscale.data_ptr(), st)
    L.launch_apply_row_shift_clamp(kints.data_ptr(), R, d, kshift.data_ptr(), 6, st)
    B = torch.empty((R, 6, W), dtype=torch.int64, device="cuda")
    L.launch_pack_bits_all_ballot_batch(kints.data_ptr(), R, d, 6, W, 0x3F, B.data_ptr(), st)
    base_k = torch.tensor([1, 2, 4, 8, 16, -32], dtype=torch.float32, device="cuda")
    Bw = (base_k[None, :] * kscale[:, None]).contiguous()
    # queries: chunk shift/scale from the floats, then the fused quantise + shift + pack
    xd = torch.from_numpy(x).cuda()
    qshift = torch.empty((Q, chunks), dtype=torch.int32, device="cuda")
    qscale = torch.empty((Q, chunks), dtype=torch.float32, device="cuda")
    L.launch_compute_chunk_shift_scale_from_input(xd.data_ptr(), 0, Q, d, chunks, 100.0, 7, 0.0, qshift.data_ptr(),
                                                  qscale.data_ptr(), st)
    A = torch.empty((Q, 7, W), dtype=torch.int64, device="cuda")
    L.launch_quantize_shift_pack_chunk_batch(xd.data_ptr(), 0, Q, d, chunks, 7, W, 0x7F, 100.0, 7, qshift.data_ptr(),
                                             A.data_ptr(), st)
    Aw = torch.tensor([1, 2, 4, 8, 16, 32, -64], dtype=torch.float32, device="cuda").repeat(Q, 1).contiguous()
    _ok(L)
    qb, kb = oracle.build_queries(x), oracle.build_keys(k)
    np.testing.assert_array_equal(A.cpu().numpy().view(np.uint64), qb["words"])
    np.testing.assert_array_equal(B.cpu().numpy().view(np.uint64), kb["words"])
    np.testing.assert_array_equal(qscale.cpu().numpy(), qb["scales"])
    np.testing.assert_array_equal(Bw.cpu().numpy(), kb["slice_weights"])
    # the dot, as batch_dot_product_multiquery_cuda_batch_caps launches it: out zero-filled, q_tile / r_tile from
    # the environment defaults, identity index arrays
    R_total = R + 8
    out = torch.zeros((Q, R_total), dtype=torch.float32, device="cuda")
    scale_inv = float(np.float32(1.0 / 10.0 ** 4))
    L.launch_popcount_weighted_keys_literal_fused_multiq(A.data_ptr(), Aw.data_ptr(), qscale.data_ptr(), chunks, 7, W,
                                                         B.data_ptr(), Bw.data_ptr(), 6, R, Q, 8, 4, None, None,
                                                         scale_inv, R_total, out.data_ptr(), st)
    torch.cuda.synchronize()
    _ok(L)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    got = out.cpu().numpy()
    np.testing.assert_array_equal(got[:, :R], want)
    assert not got[:, R:].any()                               # columns past R belong to the caller
    # without chunk scales the slice weights carry everything (the weighted kernel); a query index array is refused
    Aw_row = (Aw * 8.0).contiguous()
    L.launch_popcount_weighted_keys_literal_fused_multiq(A.data_ptr(), Aw_row.data_ptr(), None, 0, 7, W, B.data_ptr(),
                                                         Bw.data_ptr(), 6, R, Q, 8, 4, None, None, scale_inv, R_total,
                                                         out.data_ptr(), st)
    torch.cuda.synchronize()
    _ok(L)
    exact = (qb["ints"].astype(np.float64) * 8.0) @ (kb["ints"].astype(np.float64) * kb["scales"].astype(np.float64)[:, None]).T
    np.testing.assert_array_equal(out.cpu().numpy()[:, :R], exact.astype(np.float32) * np.float32(scale_inv))
    idx = torch.arange(Q, dtype=torch.int64, device="cuda")
    L.launch_popcount_weighted_keys_literal_fused_multiq(A.data_ptr(), Aw.data_ptr(), qscale.data_ptr(), chunks, 7, W,
                                                         B.data_ptr(), Bw.data_ptr(), 6, R, Q, 8, 4, None, idx.data_ptr(),
                                                         scale_inv, R_total, out.data_ptr(), st)
    assert L.bsi_launchers_last_status() == 3 and b"query index" in L.bsi_launchers_last_error()
    L.bsi_launchers_clear_status()


def test_reference_codec_sequence_through_the_launchers(launchers, oracle):
    L = launchers
    L.bsi_launchers_clear_status()
    rng = np.random.default_rng(5)
    S, W = 9, 96
    words = rng.integers(0, 2 ** 63, size=(S, W), dtype=np.uint64) * 2 + rng.integers(0, 2, size=(S, W), dtype=np.uint64)
    words[0] = 0
    words[1] = np.uint64(0xFFFFFFFFFFFFFFFF)
    words[2, 10:80] = 0
    words[3] = 0
    words[3, 17] = np.uint64(1) << np.uint64(40)
    words[4, :50] = np.uint64(0xFFFFFFFFFFFFFFFF)
    st = _st()
    wd = torch.from_numpy(words.view(np.int64)).cuda()
    counts = torch.empty((S,), dtype=torch.int64, device="cuda")
    flags = torch.empty((S,), dtype=torch.int32, device="cuda")
    sizes = torch.empty((S,), dtype=torch.int64, device="cuda")
    L.launch_slice_popcount_sum(wd.data_ptr(), S, W, counts.data_ptr(), st)
    L.launch_compress_flags_from_density(counts.data_ptr(), S, W, 0.5, flags.data_ptr(), st)
    L.launch_ewah_size(wd.data_ptr(), S, W, flags.data_ptr(), sizes.data_ptr(), st)
    off = (sizes.cumsum(0) - sizes).contiguous()
    total = int(sizes.sum().item())
    stream = torch.empty((total,), dtype=torch.int64, device="cuda")
    lens = torch.empty((S,), dtype=torch.int32, device="cuda")
    L.launch_ewah_emit(wd.data_ptr(), S, W, flags.data_ptr(), off.data_ptr(), stream.data_ptr(), lens.data_ptr(), st)
    torch.cuda.synchronize()
    _ok(L)
    want_flags = oracle.compress_flags(words, 0.5)
    want_stream, want_off, want_len = oracle.ewah_encode(words, want_flags)
    np.testing.assert_array_equal(flags.cpu().numpy(), want_flags)
    np.testing.assert_array_equal(stream.cpu().numpy().view(np.uint64), want_stream)
    np.testing.assert_array_equal(lens.cpu().numpy(), want_len)
    for s in range(S):
        back = torch.full((W,), -1, dtype=torch.int64, device="cuda")
        L.launch_ewah_decompress(stream.data_ptr() + int(want_off[s]) * 8, int(want_len[s]), W, back.data_ptr(), st)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(back.cpu().numpy().view(np.uint64), words[s])
    _ok(L)


def test_registered_keys_take_the_int8_image_route(launchers, oracle):
    """A keyset registered with bsi_launchers_register_keys: the reference's dot launcher, handed the same canonical
    planes as before, contracts the int8 image derived at registration with the image of the query planes that the
    chunk packer left -- same bits as the oracle, before and after the keyset is forgotten; planes rebuilt at the
    same address by another launcher are not served from the remembered image."""
    L = launchers
    L.bsi_launchers_register_keys.argtypes, L.bsi_launchers_register_keys.restype = [vp, i32, i32, i32, vp], i32
    L.bsi_launchers_forget_keys.argtypes, L.bsi_launchers_forget_keys.restype = [vp], i32
    L.bsi_launchers_clear_status()
    Q, R, d = 200, 300, 2048
    W, chunks = d // 64, d // 256
    rng = np.random.default_rng(77)
    st = _st()
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    kb = oracle.build_keys(k)
    B = torch.from_numpy(kb["words"].view(np.int64)).cuda()
    Bw = torch.from_numpy(kb["slice_weights"]).cuda()
    assert L.bsi_launchers_register_keys(B.data_ptr(), R, 6, W, st) == 0
    Aw = torch.tensor([1, 2, 4, 8, 16, 32, -64], dtype=torch.float32, device="cuda").repeat(Q, 1).contiguous()
    A = torch.empty((Q, 7, W), dtype=torch.int64, device="cuda")
    qshift = torch.empty((Q, chunks), dtype=torch.int32, device="cuda")
    qscale = torch.empty((Q, chunks), dtype=torch.float32, device="cuda")
    scale_inv = float(np.float32(1.0 / 10.0 ** 4))

    def build_and_dot(x):
        xd = torch.from_numpy(x).cuda()
        L.launch_compute_chunk_shift_scale_from_input(xd.data_ptr(), 0, Q, d, chunks, 100.0, 7, 0.0, qshift.data_ptr(),
                                                      qscale.data_ptr(), st)
        L.launch_quantize_shift_pack_chunk_batch(xd.data_ptr(), 0, Q, d, chunks, 7, W, 0x7F, 100.0, 7, qshift.data_ptr(),
                                                 A.data_ptr(), st)
        return dot()

    def dot():
        out = torch.zeros((Q, R), dtype=torch.float32, device="cuda")
        L.launch_popcount_weighted_keys_literal_fused_multiq(A.data_ptr(), Aw.data_ptr(), qscale.data_ptr(), chunks, 7, W,
                                                             B.data_ptr(), Bw.data_ptr(), 6, R, Q, 8, 4, None, None,
                                                             scale_inv, R, out.data_ptr(), st)
        torch.cuda.synchronize()
        _ok(L)
        return out.cpu().numpy()

    def want(x):
        qb = oracle.build_queries(x)
        return oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)[1], qb

    xs = [rng.standard_normal((Q, d)).astype(np.float32) for _ in range(2)]
    for x in xs:  # two batches through the same buffers: the remembered image follows the packer
        np.testing.assert_array_equal(build_and_dot(x), want(x)[0])
    # the same planes address refilled by another launcher (packed from integers): the image of the earlier planes is not used
    w2, qb2 = want(xs[0])
    ints = torch.from_numpy(np.ascontiguousarray(qb2["ints"])).cuda()
    L.launch_pack_bits_all_ballot_batch(ints.data_ptr(), Q, d, 7, W, 0x7F, A.data_ptr(), st)
    qscale.copy_(torch.from_numpy(qb2["scales"]).cuda())
    np.testing.assert_array_equal(dot(), w2)
    assert L.bsi_launchers_forget_keys(B.data_ptr()) == 0
    np.testing.assert_array_equal(build_and_dot(xs[1]), want(xs[1])[0])
    assert L.bsi_launchers_forget_keys(B.data_ptr()) == 0   # forgetting twice is not an error


def test_a_recorded_query_image_survives_a_larger_batch(launchers, oracle):
    """The packer and the dot of a registered keyset recorded into a HIP graph hold the address of the module's query
    image; a later, larger batch makes the module allocate a bigger image, and the recorded one must stay valid: the
    graph, replayed on new inputs afterwards (with eager work of the larger batch in between), still gives the oracle's bits."""
    L = launchers
    L.bsi_launchers_register_keys.argtypes, L.bsi_launchers_register_keys.restype = [vp, i32, i32, i32, vp], i32
    L.bsi_launchers_forget_keys.argtypes, L.bsi_launchers_forget_keys.restype = [vp], i32
    L.bsi_launchers_clear_status()
    R, d = 192, 1024
    W, chunks = d // 64, d // 256
    rng = np.random.default_rng(5150)
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    kb = oracle.build_keys(k)
    B = torch.from_numpy(kb["words"].view(np.int64)).cuda()
    Bw = torch.from_numpy(kb["slice_weights"]).cuda()
    assert L.bsi_launchers_register_keys(B.data_ptr(), R, 6, W, _st()) == 0
    scale_inv = float(np.float32(1.0 / 10.0 ** 4))

    class Batch:
        def __init__(self, Q):
            self.Q = Q
            self.x = torch.zeros((Q, d), dtype=torch.float32, device="cuda")
            self.Aw = torch.tensor([1, 2, 4, 8, 16, 32, -64], dtype=torch.float32, device="cuda").repeat(Q, 1).contiguous()
            self.A = torch.empty((Q, 7, W), dtype=torch.int64, device="cuda")
            self.qshift = torch.empty((Q, chunks), dtype=torch.int32, device="cuda")
            self.qscale = torch.empty((Q, chunks), dtype=torch.float32, device="cuda")
            self.out = torch.zeros((Q, R), dtype=torch.float32, device="cuda")

        def launch(self):
            st, Q = _st(), self.Q
            L.launch_compute_chunk_shift_scale_from_input(self.x.data_ptr(), 0, Q, d, chunks, 100.0, 7, 0.0,
                                                          self.qshift.data_ptr(), self.qscale.data_ptr(), st)
            L.launch_quantize_shift_pack_chunk_batch(self.x.data_ptr(), 0, Q, d, chunks, 7, W, 0x7F, 100.0, 7,
                                                     self.qshift.data_ptr(), self.A.data_ptr(), st)
            L.launch_popcount_weighted_keys_literal_fused_multiq(self.A.data_ptr(), self.Aw.data_ptr(), self.qscale.data_ptr(),
                                                                 chunks, 7, W, B.data_ptr(), Bw.data_ptr(), 6, R, Q, 8, 4, None,
                                                                 None, scale_inv, R, self.out.data_ptr(), st)

    def want(x):
        qb = oracle.build_queries(x)
        return oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)[1]

    small, large = Batch(96), Batch(384)
    xs = [rng.standard_normal((small.Q, d)).astype(np.float32) for _ in range(3)]
    small.x.copy_(torch.from_numpy(xs[0]))
    small.launch()                      # eager first: the image buffer of 96 rows exists
    torch.cuda.synchronize()
    _ok(L)
    np.testing.assert_array_equal(small.out.cpu().numpy(), want(xs[0]))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        small.launch()
    _ok(L)
    xl = rng.standard_normal((large.Q, d)).astype(np.float32)
    for x in xs[1:]:
        large.x.copy_(torch.from_numpy(xl))
        large.launch()                  # the first of these outgrows the recorded image
        torch.cuda.synchronize()
        _ok(L)
        np.testing.assert_array_equal(large.out.cpu().numpy(), want(xl))
        small.x.copy_(torch.from_numpy(x))
        small.out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(small.out.cpu().numpy(), want(x))
    assert L.bsi_launchers_forget_keys(B.data_ptr()) == 0
