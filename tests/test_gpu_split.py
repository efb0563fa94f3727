"""D-split launches of the int8-image dot (several workgroups per output tile, each over its own run of chunks, the
tile's last workgroup adding the partial sums) through the C ABI: bit-identical to the unsplit launch and to the
oracle's sequential chunk chain on ragged shapes, every number of segments and both tiles; tiles whose chain values
come near 2^24 units are computed again in chunk order (and the outputs then carry the chain's roundings); the
region's counters return to zero, so calls in a row, of different shapes, and replays from a HIP graph agree."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

STAT_COMBINED, STAT_RECOMPUTED, MAX_TILES = 1008, 1009, 1008


def _dev(a: np.ndarray) -> torch.Tensor:
    if a.dtype == np.uint64:
        a = a.view(np.int64)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _st():
    return torch.cuda.current_stream().cuda_stream


@pytest.fixture()
def split():
    """(library module, scratch tensor) with a fresh zeroed scratch region attached to this thread; detached, and the
    tile and split options back at their defaults, afterwards."""
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from bsipytorch_amd import _lib

    L = _lib.lib
    scratch = torch.zeros((int(L.bsi_hip_dot_split_scratch_bytes()),), dtype=torch.uint8, device="cuda")
    _lib.check(L.bsi_hip_dot_attach_split_scratch(scratch.data_ptr(), scratch.numel()), "attach")
    yield _lib, scratch
    torch.cuda.synchronize()
    _lib.check(L.bsi_hip_dot_attach_split_scratch(None, 0), "detach")
    _lib.check(L.bsi_hip_set_option(_lib.OPT_I8_SPLIT, 0), "set_option")
    _lib.check(L.bsi_hip_set_option(_lib.OPT_I8_TILE, 0), "set_option")
    from bsipytorch_amd import bsi_ops

    bsi_ops._split_tls.ptr = 0   # the module's note of what this thread has attached: nothing now


def _stats(scratch):
    words = scratch[:4096].view(torch.int32).cpu().numpy()
    return int(words[STAT_COMBINED]), int(words[STAT_RECOMPUTED]), words[:MAX_TILES]


class _Operands:
    """Device operands of one dot on the int8 images, built from the oracle's planes by the library's own layout
    kernels (checked against the oracle elsewhere)."""

    def __init__(self, hip, qb, kb, Q, R, d, Sa=7, Sb=6, image_tiled=False):
        L = hip.lib
        self.Q, self.R, self.W, self.Sa, self.Sb = Q, R, (d + 63) // 64, Sa, Sb
        self.chunks = (self.W + 3) // 4
        self.A = _dev(qb["words"])
        self.scales = _dev(qb["scales"])
        self.stride = self.chunks if qb["chunk_scale"] else 1
        self.B = _dev(kb["words"])
        self.Bw = _dev(kb["slice_weights"])
        self.A8 = torch.zeros((Q, self.chunks * 256), dtype=torch.int8, device="cuda")
        hip.check(L.bsi_hip_planes_to_int8(self.A.data_ptr(), Q, Sa, self.W, self.A8.data_ptr(), _st()), "query image")
        self.layout = 3 if image_tiled else 2
        if image_tiled:   # the image in tiles of 64 rows x half-chunks
            self.K8 = torch.full((int(L.bsi_hip_int8_tiled_bytes(R, self.W)),), 77, dtype=torch.int8, device="cuda")
            hip.check(L.bsi_hip_planes_to_int8_tiled(self.B.data_ptr(), R, Sb, self.W, self.K8.data_ptr(), _st()), "key image")
        else:
            self.K8 = torch.full((R, self.chunks * 256), 77, dtype=torch.int8, device="cuda")
            hip.check(L.bsi_hip_planes_to_int8(self.B.data_ptr(), R, Sb, self.W, self.K8.data_ptr(), _st()), "key image")

    def dot(self, hip, bias=None, R_total=None):
        L = hip.lib
        R_total = self.R if R_total is None else R_total
        out = torch.full((self.Q, R_total), float("nan"), dtype=torch.float32, device="cuda")
        args = (self.A.data_ptr(), self.A8.data_ptr(), self.scales.data_ptr(), self.stride, self.Sa, self.W,
                self.K8.data_ptr(), self.layout, self.Bw.data_ptr(), self.Sb, self.R, self.Q, float(np.float32(1e-4)), R_total)
        if bias is None:
            hip.check(L.bsi_hip_dot(*args, out.data_ptr(), None, hip.CORE_MFMA, None, 0, _st()), "dot")
        else:
            hip.check(L.bsi_hip_dot_bias(*args, bias.data_ptr(), out.data_ptr(), hip.CORE_MFMA, None, 0, _st()), "dot_bias")
        torch.cuda.synchronize()
        return out.cpu().numpy()


def _case(oracle, Q, R, d, seed, relu=False):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((Q, d)).astype(np.float32)
    if relu:
        x = np.maximum(x, 0)
    x[:, rng.permutation(d)[:2]] *= 20.0   # two outlier columns: their chunks get larger scales
    x[1, :256] = 0.0                       # an all-zero chunk
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    k[R // 2] *= 50                        # one key row with a large shift
    qb, kb = oracle.build_queries(x, 2, 7), oracle.build_keys(k, 2, 6)
    _, out = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    return qb, kb, out


def _tiles(Q, R, tile):
    return ((R + 127) // 128) * ((Q + (127 if tile == 128 else 63)) // (128 if tile == 128 else 64))


@pytest.mark.parametrize("Q,R,d,relu", [(200, 300, 2048, False), (130, 129, 4352, True), (64, 128, 1024, False),
                                       (257, 250, 3072, False)])
@pytest.mark.parametrize("tile", [128, 12864])
@pytest.mark.parametrize("segments", [2, 3, 4, 8])
def test_split_equals_the_unsplit_launch_and_the_oracle(split, oracle, Q, R, d, relu, tile, segments):
    hip, scratch = split
    L = hip.lib
    qb, kb, want = _case(oracle, Q, R, d, seed=Q + R + d, relu=relu)
    ops = _Operands(hip, qb, kb, Q, R, d)
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_SPLIT, 1), "set_option")   # never split
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, tile), "set_option")
    unsplit = ops.dot(hip)
    assert _stats(scratch)[:2] == (0, 0)
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_SPLIT, segments), "set_option")
    t, s = ctypes.c_int(0), ctypes.c_int(0)
    hip.check(L.bsi_hip_dot_split_plan(R, Q, ops.W, ctypes.byref(t), ctypes.byref(s)), "plan")
    assert (t.value, s.value) == (tile, min(segments, ops.chunks))
    got = ops.dot(hip)
    combined, recomputed, counters = _stats(scratch)
    assert (combined, recomputed) == (_tiles(Q, R, tile), 0)   # every tile went the partial-sum way
    assert not counters.any()                                  # and left its counter at zero
    np.testing.assert_array_equal(got, unsplit)
    np.testing.assert_array_equal(got, want)
    # with a bias in the epilogue and a row stride, as a layer calls it
    bias = torch.linspace(-3, 3, R, device="cuda")
    got_b = ops.dot(hip, bias=bias, R_total=R + 5)
    np.testing.assert_array_equal(got_b[:, :R], want + bias.cpu().numpy()[None, :])
    assert np.isnan(got_b[:, R:]).all()


@pytest.mark.parametrize("Sa,Sb", [(7, 6), (8, 8), (4, 3), (2, 5)])
@pytest.mark.parametrize("image_tiled", [False, True])
def test_split_on_other_bit_widths_and_the_tiled_key_image(split, oracle, Sa, Sb, image_tiled):
    """The exactness limit follows the operands' widths (the accumulators carry 2^(16 - Sa - Sb) times the integers),
    and a segment's run of chunks is addressed in the tiled key image as in the row-major one."""
    hip, scratch = split
    L = hip.lib
    Q, R, d = 150, 260, 2560
    rng = np.random.default_rng(Sa * 10 + Sb)
    x = rng.standard_normal((Q, d)).astype(np.float32)
    x[:, 7] *= 30.0
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    qb, kb = oracle.build_queries(x, 2, Sa), oracle.build_keys(k, 2, Sb)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    ops = _Operands(hip, qb, kb, Q, R, d, Sa, Sb, image_tiled)
    for tile, segments in ((128, 5), (12864, 2), (12864, 10)):
        hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, tile), "set_option")
        hip.check(L.bsi_hip_set_option(hip.OPT_I8_SPLIT, segments), "set_option")
        before = _stats(scratch)[0]
        np.testing.assert_array_equal(ops.dot(hip), want)
        assert _stats(scratch)[0] - before == _tiles(Q, R, tile) and _stats(scratch)[1] == 0


def _rounding_case(oracle, Q, R, chunks, seed, big_queries):
    """Same-sign products with mixed power-of-two scales: the chain of the rows in big_queries passes 2^24 units and
    rounds, so only the chunk order reproduces their bits; the other rows stay small."""
    rng = np.random.default_rng(seed)
    d = 256 * chunks
    a = rng.integers(-3, 4, size=(Q, d)).astype(np.int64)
    a[big_queries] = rng.integers(40, 64, size=(len(big_queries), d))
    b = rng.integers(20, 32, size=(R, d)).astype(np.int64)
    scales = np.ones((Q, chunks), np.float32)
    scales[big_queries] = (2.0 ** rng.integers(0, 8, size=(len(big_queries), chunks))).astype(np.float32)
    bscale = (2.0 ** rng.integers(0, 5, size=R)).astype(np.float32)
    qb = dict(words=oracle.pack(a, 7), scales=scales, chunk_scale=True)
    kb = dict(words=oracle.pack(b, 6), slice_weights=(oracle.slice_weights(6)[None] * bscale[:, None]).astype(np.float32))
    ints, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], bscale, np.float32(1e-4))
    return qb, kb, ints, want, d


@pytest.mark.parametrize("tile", [128, 12864])
@pytest.mark.parametrize("segments", [2, 4, 5])
def test_tiles_whose_chain_could_round_are_computed_again_in_chunk_order(split, oracle, tile, segments):
    hip, scratch = split
    L = hip.lib
    Q, R, chunks = 260, 140, 40
    big = list(range(128, 140))  # queries of the second 128-row tile (and of the third 64-row tile) only
    qb, kb, ints, want, d = _rounding_case(oracle, Q, R, chunks, seed=11, big_queries=big)
    # the case does what it is meant to: the big rows' exact sums pass 2^24 and are not what the fp32 chain gives
    exact = (ints.astype(np.float64) * qb["scales"][:, None, :].astype(np.float64)).sum(-1)
    assert np.abs(exact[big]).max() > 2.0 ** 24 and np.abs(np.delete(exact, big, axis=0)).max() < 2.0 ** 20
    ops = _Operands(hip, qb, kb, Q, R, d)
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_TILE, tile), "set_option")
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_SPLIT, segments), "set_option")
    got = ops.dot(hip)
    combined, recomputed, counters = _stats(scratch)
    key_tiles = (R + 127) // 128
    assert recomputed == key_tiles                       # the query tile that holds the big rows, for every key tile
    assert combined == _tiles(Q, R, tile) - key_tiles    # the others by partial sums
    assert not counters.any()
    np.testing.assert_array_equal(got, want)
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_SPLIT, 1), "set_option")
    np.testing.assert_array_equal(ops.dot(hip), want)


def test_calls_in_a_row_share_one_region(split, oracle):
    """Shapes of different tile counts one after the other on the same region, the second smaller, then the first
    again: every launch finds the counters at zero."""
    hip, scratch = split
    L = hip.lib
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_SPLIT, 4), "set_option")
    cases = []
    for Q, R, d in [(300, 520, 2048), (70, 100, 1024), (300, 520, 2048)]:
        qb, kb, want = _case(oracle, Q, R, d, seed=Q + d)
        cases.append((_Operands(hip, qb, kb, Q, R, d), want))
    for _ in range(3):
        for ops, want in cases:
            np.testing.assert_array_equal(ops.dot(hip), want)
    combined, recomputed, counters = _stats(scratch)
    assert combined == 3 * (2 * _tiles(300, 520, 128) + _tiles(70, 100, 128)) and recomputed == 0 and not counters.any()


def test_the_choice_by_cost(split):
    """The launch plan.  Partial sums travel through memory, which costs several microseconds: the shapes of the
    scope table stay unsplit (their small-tile launches are faster, measured), grids of a few tiles over long rows
    split; nothing splits without a region or with the option at 1."""
    hip, scratch = split
    L = hip.lib
    t, s = ctypes.c_int(0), ctypes.c_int(0)

    def plan(R, Q, d):
        hip.check(L.bsi_hip_dot_split_plan(R, Q, d // 64, ctypes.byref(t), ctypes.byref(s)), "plan")
        return t.value, s.value

    assert plan(2048, 512, 8192) == (64, 1)      # FC2-like
    assert plan(8192, 512, 2048) == (128, 1)     # the headline shape: 256 tiles fill the GPU
    assert plan(256, 64, 2048)[1] == 1           # correctness scale
    assert plan(4096, 128, 16384)[1] == 1 and plan(1024, 128, 8192)[1] == 1
    assert plan(512, 128, 16384) == (12864, 6)   # 8 tiles of 128 x 64 over 64 chunks
    assert plan(256, 64, 32768) == (12864, 8)
    tile, segs = plan(1024, 256, 16384)
    assert tile == 12864 and 3 <= segs <= 6
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_SPLIT, 1), "set_option")
    assert plan(512, 128, 16384) == (6432, 1)
    hip.check(L.bsi_hip_set_option(hip.OPT_I8_SPLIT, 0), "set_option")
    hip.check(L.bsi_hip_dot_attach_split_scratch(None, 0), "detach")
    assert plan(512, 128, 16384) == (6432, 1)
    # a region too small for the partial sums of a choice is not used for it
    hip.check(L.bsi_hip_dot_attach_split_scratch(scratch.data_ptr(), 4096 + 128 * 64 * 4 * 8 * 3), "attach")
    assert plan(512, 128, 16384) == (12864, 3)
    hip.check(L.bsi_hip_dot_attach_split_scratch(scratch.data_ptr(), 4096 + 128 * 64 * 4 * 8), "attach")
    assert plan(512, 128, 16384) == (6432, 1)
    assert L.bsi_hip_dot_attach_split_scratch(scratch.data_ptr() + 8, 1 << 20) == 1
    assert L.bsi_hip_dot_attach_split_scratch(scratch.data_ptr(), 4096) == 1


def test_split_launches_replay_from_a_hip_graph():
    """A few-tiles, long-rows dot through bsi_ops (build + dot on the split kernel) recorded once and replayed with new
    inputs, eager work and synchronisations between the replays: every replay equals the eager result."""
    import os

    from bsipytorch_amd import _lib, bsi_ops

    assert os.environ.get("BSI_DOT_SPLIT", "1") != "0"
    torch.manual_seed(5)
    Q, R, D = 128, 512, 16384
    kcap, *_ = bsi_ops.build_bsi_keys_cuda(torch.randn(R, D) * 0.02, 2, 0.5)
    xs = [torch.relu(torch.randn(Q, D)).cuda() for _ in range(3)]

    def run(x):
        qcap = bsi_ops.build_bsi_queries_cuda_batch_packed(x, 2, 0.5)
        return bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)[0]

    eager = [run(x).clone() for x in xs]
    t, s = ctypes.c_int(0), ctypes.c_int(0)
    _lib.check(_lib.lib.bsi_hip_dot_split_plan(R, Q, D // 64, ctypes.byref(t), ctypes.byref(s)), "plan")
    assert s.value >= 2, "this shape is meant to take the split route"
    static_x = xs[0].clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        static_out = run(static_x)
    for rep in range(2):
        for x, want in zip(xs, eager):
            static_x.copy_(x)
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_out, want)
            assert torch.equal(run(x), want)   # eager work between the replays, on its own region
    _lib.check(_lib.lib.bsi_hip_dot_attach_split_scratch(None, 0), "detach")
    bsi_ops._split_tls.ptr = 0
