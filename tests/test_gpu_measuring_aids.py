"""The library's measuring aids through the C ABI: device info, the timed dot (same bits as the untimed one, a
plausible duration), the peak probes (finite rates within the machine's published limits) and the timeline read
(refused by the ordinary build, served by the timeline build when that library is present)."""
import ctypes
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture()
def ops(monkeypatch):
    from bsipytorch_amd import bsi_ops

    for k in list(os.environ):
        if k.startswith("BSI_"):
            monkeypatch.delenv(k)
    bsi_ops._reset_flag_cache()
    yield bsi_ops
    bsi_ops._reset_flag_cache()


def test_device_info_and_version(ops):
    from bsipytorch_amd import _lib

    arch = ctypes.create_string_buffer(64)
    cus, lds = ctypes.c_int(0), ctypes.c_int(0)
    _lib.check(_lib.lib.bsi_hip_device_info(arch, 64, ctypes.byref(cus), ctypes.byref(lds)), "bsi_hip_device_info")
    assert arch.value.decode().startswith("gfx950")
    assert cus.value == torch.cuda.get_device_properties(0).multi_processor_count
    assert lds.value >= 160 * 1024  # the int8-image kernel's ring needs 128 KiB + scales of one workgroup
    assert "gfx950" in _lib.version()
    # a buffer too small for the name gets its terminated beginning
    small = ctypes.create_string_buffer(b"xxxxxxxx", 8)
    _lib.check(_lib.lib.bsi_hip_device_info(small, 4, ctypes.byref(cus), ctypes.byref(lds)), "bsi_hip_device_info")
    assert small.raw[:4] == b"gfx\0" and small.raw[4:] == b"xxxx"


@pytest.mark.parametrize("Q,R,D,core", [(64, 256, 2048, "mfma"), (5, 100, 512, "auto"), (32, 64, 256, "valu")])
def test_timed_dot_gives_the_bits_of_the_untimed_dot(ops, oracle, Q, R, D, core):
    from bsipytorch_amd import _lib

    torch.manual_seed(Q * 7 + R)
    K = torch.randn(R, D) * 0.02
    X = torch.randn(Q, D)
    kcap, *_ = ops.build_bsi_keys_cuda(K, 2, 0.5)
    qcap = ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.5)
    ref, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    W = (D + 63) // 64
    chunks = (W + 3) // 4
    code = {"auto": _lib.CORE_AUTO, "mfma": _lib.CORE_MFMA, "valu": _lib.CORE_VALU}[core]
    ws_bytes = int(_lib.lib.bsi_hip_dot_workspace_bytes(Q, W, code))
    ws = torch.empty((max(ws_bytes, 16),), dtype=torch.uint8, device="cuda")
    out = torch.full((Q, R), float("nan"), dtype=torch.float32, device="cuda")
    kptr, klayout = ops.key_operand(kcap, Q, qcap.Sa, code)
    us = ctypes.c_float(-1.0)
    args = (qcap.words.data_ptr(), qcap.ints8.data_ptr(), qcap.chunk_scales.data_ptr(), chunks, qcap.Sa, W, kptr, klayout,
            kcap.slice_weights.data_ptr(), kcap.Sb, R, Q, float(oracle.scale_inv(2, 2)), R, out.data_ptr(), code, ws.data_ptr(), ws_bytes)
    st = torch.cuda.current_stream().cuda_stream
    _lib.check(_lib.lib.bsi_hip_dot_timed(*args, 7, ctypes.byref(us), st), "bsi_hip_dot_timed")
    assert 0.5 < us.value < 5000.0  # microseconds per launch: above the launch floor, far below a stall
    if core != "valu":  # the popcount core is a different kernel than the dispatcher's choice; same integers, same chain
        assert torch.equal(out.cpu(), ref.cpu())
    # against the oracle on the quantised operands
    qb, kb = oracle.build_queries(X.numpy(), 2, 7), oracle.build_keys(K.numpy(), 2, 6)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), np.asarray(want, dtype=np.float32).view(np.uint32))
    # iters < 1 is refused
    assert _lib.lib.bsi_hip_dot_timed(*args, 0, ctypes.byref(us), st) != 0


def test_peak_probes_report_rates_within_the_machine(ops):
    from bsipytorch_amd import _lib

    st = torch.cuda.current_stream().cuda_stream
    v = ctypes.c_double(0.0)
    _lib.check(_lib.lib.bsi_hip_probe_valu_popcount(ctypes.byref(v), st), "bsi_hip_probe_valu_popcount")
    # lane operations per second of the v_and / v_bcnt pair: 256 CUs x 64 lanes x <= 2.4 GHz x at most 2 per cycle
    assert 1e12 < v.value < 256 * 64 * 2.4e9 * 2
    _lib.check(_lib.lib.bsi_hip_probe_mfma_i8(ctypes.byref(v), st), "bsi_hip_probe_mfma_i8")
    assert 1e15 < v.value <= 5.1e15  # int8 ops per second: above a fifth of, and not above, the published 5.0 POP/s
    ceiling = v.value
    _lib.check(_lib.lib.bsi_hip_probe_mfma_i8_operands(1, ctypes.byref(v), st), "bsi_hip_probe_mfma_i8_operands")
    assert 1e15 < v.value <= ceiling * 1.05  # random operands switch more: never faster than near-constant ones
    assert _lib.lib.bsi_hip_probe_mfma_i8_operands(2, ctypes.byref(v), st) != 0
    buf = torch.empty((256 << 20,), dtype=torch.uint8, device="cuda")
    buf.zero_()
    _lib.check(_lib.lib.bsi_hip_probe_stream_read(buf.data_ptr(), buf.numel(), ctypes.byref(v), st), "bsi_hip_probe_stream_read")
    assert 1e12 < v.value < 8.1e12  # bytes per second from HBM: above 1 TB/s, not above the published 8 TB/s
    rates = []
    for pattern in range(4):
        _lib.check(_lib.lib.bsi_hip_probe_l2_to_lds(buf.data_ptr(), buf.numel(), pattern, ctypes.byref(v), st),
                   "bsi_hip_probe_l2_to_lds")
        rates.append(v.value)
        # bytes per second from L2 into LDS over all CUs: at most 64 bytes per cycle and CU at 2.4 GHz
        assert 5e12 < v.value < 256 * 64 * 2.4e9 * 1.02
    assert _lib.lib.bsi_hip_probe_l2_to_lds(buf.data_ptr(), buf.numel(), 4, ctypes.byref(v), st) != 0  # no such pattern
    assert _lib.lib.bsi_hip_probe_l2_to_lds(buf.data_ptr(), 4096, 0, ctypes.byref(v), st) != 0        # region too small
    assert _lib.lib.bsi_hip_probe_stream_read(None, 1 << 20, ctypes.byref(v), st) != 0


def test_timeline_read_is_refused_by_the_ordinary_build_and_served_by_the_timeline_build(ops):
    from bsipytorch_amd import _lib

    stamps = (ctypes.c_ulonglong * (8 * 4))()
    assert _lib.lib.bsi_hip_timeline_read(stamps, 4) != 0
    assert "timeline" in _lib.lib.bsi_hip_last_error().decode().lower()
    path = os.path.join(os.path.dirname(_lib.LIB_PATH), "libbsi_hip_timeline.so")
    if not os.path.exists(path) or os.path.samefile(path, _lib.LIB_PATH):
        pytest.skip("the timeline build of the library is not present")
    tl = ctypes.CDLL(path)
    missing = [name for name in _lib.PROTOTYPES if not hasattr(tl, name)]
    if missing:
        pytest.skip(f"the timeline build present is older than the library (no {missing[0]}): rebuild it with make TIMELINE=1")
    for name, argtypes in _lib.PROTOTYPES.items():
        fn = getattr(tl, name)
        fn.argtypes = argtypes
        fn.restype = _lib._RESTYPES.get(name, ctypes.c_int)
    # one int8-image dot through the timeline library (operands built by the ordinary one: same layouts)
    Q, R, D = 128, 256, 1024
    torch.manual_seed(3)
    K = torch.randn(R, D) * 0.02
    X = torch.randn(Q, D)
    kcap, *_ = ops.build_bsi_keys_cuda(K, 2, 0.5)
    qcap = ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.5)
    ref, *_ = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)
    W, chunks = D // 64, D // 256
    kptr, klayout = ops.key_operand(kcap, Q, qcap.Sa, _lib.CORE_MFMA)
    out = torch.empty((Q, R), dtype=torch.float32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    rc = tl.bsi_hip_dot(qcap.words.data_ptr(), qcap.ints8.data_ptr(), qcap.chunk_scales.data_ptr(), chunks, qcap.Sa, W, kptr,
                        klayout, kcap.slice_weights.data_ptr(), kcap.Sb, R, Q, 1e-4, R, out.data_ptr(), None,
                        _lib.CORE_MFMA, None, 0, st)
    assert rc == 0, tl.bsi_hip_last_error().decode()
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), ref.cpu())  # the stamps change no result
    n = 2
    stamps = (ctypes.c_ulonglong * (8 * n))()
    assert tl.bsi_hip_timeline_read(stamps, n) == 0, tl.bsi_hip_last_error().decode()
    s = np.array(list(stamps), dtype=np.uint64).reshape(n, 8)
    assert (s > 0).all()
    # per workgroup: MFMA wave entered <= first stage in LDS <= chunk loop done <= outputs stored; the loader wave
    # entered <= its first load issued <= three stages issued <= loader done
    for wg in s:
        assert wg[0] <= wg[1] <= wg[2] <= wg[3]
        assert wg[4] <= wg[6] <= wg[7] <= wg[5]
    # the read cleared them
    assert tl.bsi_hip_timeline_read(stamps, n) == 0
    assert not any(stamps)
