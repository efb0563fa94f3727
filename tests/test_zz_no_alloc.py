"""bsi_hip_dot_static_scratch (the dot that allocates nothing: its int8 query operands go into an array inside the
library's device image) against bsi_hip_dot with a caller's workspace, through the C ABI: bit-identical outputs and
integer accumulators on two calls in a row, the second with a smaller input (the array keeps the first call's bytes),
on every key layout the matrix-core dot reads; also against the oracle, and the size limit's error."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 8 << 20


def _dev(a: np.ndarray) -> torch.Tensor:
    if a.dtype == np.uint64:
        a = a.view(np.int64)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _st():
    return torch.cuda.current_stream().cuda_stream


def _case(oracle, Q, R, d, seed, relu=False):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((Q, d)).astype(np.float32)
    if relu:
        x = np.maximum(x, 0)
    x[:, rng.permutation(d)[:2]] *= 20.0
    k = (rng.standard_normal((R, d)) * 0.02).astype(np.float32)
    k[R // 2] *= 50
    qb, kb = oracle.build_queries(x, 2, 7), oracle.build_keys(k, 2, 6)
    ints, out = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2))
    return qb, kb, ints, out


def _key_operand(L, hip, kb, R, W, layout):
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


def _both(L, hip, qb, kb, Q, R, d, layout, want_ints):
    """(ints, out) of bsi_hip_dot with a workspace and of bsi_hip_dot_static_scratch on the same operands."""
    W = (d + 63) // 64
    chunks = (W + 3) // 4
    A, scales, Bw = _dev(qb["words"]), _dev(qb["scales"]), _dev(kb["slice_weights"])
    stride = chunks if qb["chunk_scale"] else 1
    B = _key_operand(L, hip, kb, R, W, layout)
    scale_inv = float(np.float32(1e-4))
    res = []
    for static in (False, True):
        out = torch.full((Q, R), float("nan"), dtype=torch.float32, device="cuda")
        ints = torch.full((Q, R, chunks), -7, dtype=torch.int32, device="cuda") if want_ints else None
        ip = ints.data_ptr() if ints is not None else None
        if static:
            hip.check(L.bsi_hip_dot_static_scratch(A.data_ptr(), scales.data_ptr(), stride, 7, W, B.data_ptr(), layout,
                                                   Bw.data_ptr(), 6, R, Q, scale_inv, R, out.data_ptr(), ip, _st()),
                      "bsi_hip_dot_static_scratch")
        else:
            nbytes = int(L.bsi_hip_dot_workspace_bytes(Q, W, 2))
            ws = torch.full((nbytes,), 0x33, dtype=torch.uint8, device="cuda")
            hip.check(L.bsi_hip_dot(A.data_ptr(), None, scales.data_ptr(), stride, 7, W, B.data_ptr(), layout,
                                    Bw.data_ptr(), 6, R, Q, scale_inv, R, out.data_ptr(), ip, 2, ws.data_ptr(), nbytes,
                                    _st()), "bsi_hip_dot")
        torch.cuda.synchronize()
        res.append((ints.cpu().numpy() if ints is not None else None, out.cpu().numpy()))
    return res


@pytest.mark.parametrize("layout", [2, 1, 0])   # int8 key image, tiled planes, canonical planes
@pytest.mark.parametrize("want_ints", [False, True])
def test_static_scratch_dot_matches_workspace_dot_twice(oracle, layout, want_ints):
    from bsipytorch_amd import _lib as hip

    L = hip.lib
    # first call: many rows (2.6 MiB of int8 operands); second: fewer and shorter rows, so most of the array still
    # holds the first call's bytes; third: a few rows (the plane-streaming kernel on the tiled layout)
    for Q, R, d, relu in [(330, 200, 8192, True), (70, 150, 1024, False), (5, 90, 2048, False)]:
        qb, kb, want_ints_arr, want_out = _case(oracle, Q, R, d, seed=Q + d, relu=relu)
        (ints_w, out_w), (ints_s, out_s) = _both(L, hip, qb, kb, Q, R, d, layout, want_ints)
        np.testing.assert_array_equal(out_s, out_w)
        np.testing.assert_array_equal(out_s, want_out)
        if want_ints:
            np.testing.assert_array_equal(ints_s, ints_w)
            np.testing.assert_array_equal(ints_s, want_ints_arr)


def test_static_scratch_dot_rejects_what_does_not_fit():
    from bsipytorch_amd import _lib as hip

    L = hip.lib
    Q, W = 1025, 128                               # 1025 x 8192 bytes: one row too many for 8 MiB
    assert Q * (W // 4) * 256 > SCRATCH_BYTES
    t = torch.zeros(64, dtype=torch.int64, device="cuda")  # never read: the size check comes first
    rc = L.bsi_hip_dot_static_scratch(t.data_ptr(), t.data_ptr(), W // 4, 7, W, t.data_ptr(), 2, t.data_ptr(), 6, 16, Q,
                                      1.0, 16, t.data_ptr(), None, _st())
    assert rc == 1 and b"static scratch" in L.bsi_hip_last_error()
    rc = L.bsi_hip_dot_static_scratch(None, t.data_ptr(), 1, 7, 4, t.data_ptr(), 2, t.data_ptr(), 6, 16, 16, 1.0, 16,
                                      t.data_ptr(), None, _st())
    assert rc == 1


def test_static_scratch_dot_replays_from_a_captured_graph(oracle):
    """After one eager call of the shape class (which looks the array's address up and opts the kernels in to their
    LDS), the entry point is recorded into a HIP graph and replayed several times with new query planes copied in and
    eager work between the replays: every replay equals the eager result and the oracle."""
    from bsipytorch_amd import _lib as hip

    L = hip.lib
    Q, R, d = 130, 200, 2048
    W, chunks = d // 64, d // 256
    cases = [_case(oracle, Q, R, d, seed=s) for s in (1, 2, 3)]
    kb = cases[0][1]
    B = _key_operand(L, hip, kb, R, W, 2)
    Bw = _dev(kb["slice_weights"])
    A, scales = _dev(cases[0][0]["words"]).clone(), _dev(cases[0][0]["scales"]).clone()
    out = torch.full((Q, R), float("nan"), dtype=torch.float32, device="cuda")
    scale_inv = float(np.float32(1e-4))

    def call(stream):
        hip.check(L.bsi_hip_dot_static_scratch(A.data_ptr(), scales.data_ptr(), chunks, 7, W, B.data_ptr(), 2, Bw.data_ptr(), 6,
                                               R, Q, scale_inv, R, out.data_ptr(), None, stream), "bsi_hip_dot_static_scratch")

    call(_st())                       # the warm-up call, outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call(torch.cuda.current_stream().cuda_stream)
    for rep in range(2):
        for qb, kb_i, _, _ in cases:
            # every case against the first case's keys
            _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
            A.copy_(_dev(qb["words"]))
            scales.copy_(_dev(qb["scales"]))
            out.fill_(float("nan"))
            g.replay()
            torch.cuda.synchronize()
            np.testing.assert_array_equal(out.cpu().numpy(), want)
            other = torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")  # eager work in between
            torch.cuda.synchronize()
            del other
