"""CPU-side checks of the C-ABI library and the host logic (no kernel is launched here)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "bsi_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bsi_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from bsipytorch_amd import _lib

    names = _declared_symbols()
    assert len(names) >= 25
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"libbsi_hip.so does not export {n}"
    assert set(names) == set(_lib.PROTOTYPES), set(names) ^ set(_lib.PROTOTYPES)
    assert "gfx950" in _lib.version()


def test_argument_validation_returns_error_codes():
    from bsipytorch_amd import _lib

    L = _lib.lib
    # W64 = 0 is rejected before anything touches the device
    rc = L.bsi_hip_dot(None, None, None, 8, 7, 0, None, 0, None, 6, 4, 4, 1.0, 4, None, None, 0, None, 0, None)
    assert rc == 1 and b"W64" in L.bsi_hip_last_error()
    rc = L.bsi_hip_dot(None, None, None, 8, 7, 32, None, 0, None, 6, 4, -1, 1.0, 4, None, None, 0, None, 0, None)
    assert rc == 1
    # stride must be chunks or 1
    rc = L.bsi_hip_dot(1, None, 1, 3, 7, 32, 1, 0, 1, 6, 4, 4, 1.0, 4, 1, None, 0, None, 0, None)
    assert rc == 1 and b"stride" in L.bsi_hip_last_error()
    rc = L.bsi_hip_dot(1, None, 1, 8, 7, 32, 1, 0, 1, 6, 8, 4, 1.0, 4, 1, None, 0, None, 0, None)
    assert rc == 1 and b"R_total" in L.bsi_hip_last_error()
    rc = L.bsi_hip_build_fixed(None, 0, 4, 4, 2, 1, 1, 0.0, None, None, None, None, None)
    assert rc == 1 and b"fixed_bits" in L.bsi_hip_last_error()
    rc = L.bsi_hip_planes_to_int8(None, 4, 9, 4, None, None)
    assert rc == 1
    # rows longer than the matrix-core kernels' 32-bit operand offsets reach are refused when that core is forced
    W_long = 4 * 32769
    rc = L.bsi_hip_dot(1, None, 1, 1, 7, W_long, 1, 0, 1, 6, 4, 4, 1.0, 4, 1, None, _lib.CORE_MFMA, None, 0, None)
    assert rc == 3 and b"chunks" in L.bsi_hip_last_error()
    # more query rows than the launch grid's second dimension holds tiles of 32 for: refused as an argument error
    too_many = 65535 * 32 + 1
    rc = L.bsi_hip_dot(1, None, 1, 8, 7, 32, 1, 0, 1, 6, 4, too_many, 1.0, 4, 1, None, 0, None, 0, None)
    assert rc == 1 and b"query rows per call" in L.bsi_hip_last_error()
    # empty problems are fine and launch nothing
    assert L.bsi_hip_dot(None, None, None, 8, 7, 32, None, 0, None, 6, 0, 0, 1.0, 0, None, None, 0, None, 0, None) == 0
    assert L.bsi_hip_build_fixed(None, 0, 0, 128, 2, 7, 1, 0.0, None, None, None, None, None) == 0
    assert L.bsi_hip_dot_workspace_bytes(512, 32, _lib.CORE_MFMA) == 512 * 8 * 256
    assert L.bsi_hip_dot_workspace_bytes(512, 32, _lib.CORE_VALU) == 0
    with pytest.raises(_lib.BsiHipError):
        _lib.check(rc=1, what="x")


def test_flags_defaults_and_overrides(monkeypatch):
    from bsipytorch_amd import bsi_ops

    for k in list(os.environ):
        if k.startswith("BSI_"):
            monkeypatch.delenv(k)
    bsi_ops._reset_flag_cache()
    f = dict(bsi_ops._flags())
    assert (f["bits_q"], f["bits_k"], f["chunk_scale"], f["clip_k"], f["profile"]) == (7, 6, True, 0.0, False)
    monkeypatch.setenv("BSI_FIXED_BITS", "5")
    monkeypatch.setenv("BSI_FIXED_BITS_KEYS", "1")   # clamped up to 2
    monkeypatch.setenv("BSI_FIXED_CHUNK_SCALE", "0")
    monkeypatch.setenv("BSI_FIXED_CLIP_K", "6.5")
    monkeypatch.setenv("BSI_DOT_CORE", "valu")
    bsi_ops._reset_flag_cache()
    f = dict(bsi_ops._flags())
    assert (f["bits_q"], f["bits_k"], f["chunk_scale"], f["clip_k"]) == (5, 2, False, 6.5)
    assert f["core"] == 1
    monkeypatch.setenv("BSI_FIXED_BITS_QUERIES", "0")
    bsi_ops._reset_flag_cache()
    assert bsi_ops._flags()["bits_q"] == 0   # decimal mode for queries; keys stay fixed
    assert bsi_ops._flags()["bits_k"] == 2
    for k in ("BSI_FIXED_BITS", "BSI_FIXED_BITS_KEYS", "BSI_FIXED_CHUNK_SCALE", "BSI_FIXED_CLIP_K", "BSI_DOT_CORE",
              "BSI_FIXED_BITS_QUERIES"):
        monkeypatch.delenv(k)
    bsi_ops._reset_flag_cache()


def test_module_surface_matches_reference_names():
    import bsi_ops  # the drop-in name

    gpu = ["build_bsi_keys_cuda", "build_bsi_queries_cuda_batch_packed", "build_bsi_queries_cuda_batch",
           "build_bsi_query_cuda", "build_bsi_query_cuda_hybrid", "batch_dot_product_multiquery_cuda_batch_caps",
           "batch_dot_product_multiquery_cuda_caps", "bsi_keys_cuda_stats", "bsi_query_caps_stats",
           "get_last_query_build_profile_cuda", "reset_last_query_build_profile_cuda", "cuda_builder_version"]
    cpu = ["dot_product", "dot_product_decimal", "vector_dot_product", "vector_dot_product_no_precison",
           "random_number_dot_product_vector", "random_number_dot_product_bsi", "batch_dot_product", "build_bsi_keys",
           "build_bsi_query", "batch_dot_product_prebuilt", "batch_dot_product_prebuilt_capsule",
           "keyset_slice_stats", "tensor_slice_stats", "keyset_size_on_disk", "save_keyset", "debug_bsi_query_words"]
    for n in gpu + cpu + ["debug_quantize_int64_cpu", "CUDA_BUILDER_VERSION"]:
        assert hasattr(bsi_ops, n), n
    # the scalar entry points run on the device kernels too: without a GPU they refuse, they do not fall back
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="no GPU visible"):
            bsi_ops.dot_product(torch.zeros(2), torch.zeros(2), 10.0)
        with pytest.raises(RuntimeError, match="no GPU visible"):
            bsi_ops.batch_dot_product(torch.zeros(2), torch.zeros(3, 2), 2)
        with pytest.raises(RuntimeError, match="no GPU visible"):
            bsi_ops.tensor_slice_stats(torch.zeros(2), 2)
    with pytest.raises(RuntimeError, match="must be 2D"):
        bsi_ops.build_bsi_keys(torch.zeros(2), 2)
    with pytest.raises(RuntimeError, match="Invalid BSI keys capsule"):
        bsi_ops.keyset_slice_stats(object())
    assert bsi_ops.PrebuiltBSIKeys.name == "PrebuiltBSIKeys" and bsi_ops.PrebuiltBSIQuery.name == "PrebuiltBSIQuery"
    assert bsi_ops.get_last_query_build_profile_cuda() == (0, 0, 0)
    assert bsi_ops.PrebuiltBSIKeysCUDA.name == "PrebuiltBSIKeysCUDA"
    assert bsi_ops.PrebuiltBSIQueryBatchCUDA.name == "PrebuiltBSIQueryBatchCUDA"
    assert bsi_ops.PrebuiltBSIQueryCUDA.name == "PrebuiltBSIQueryCUDA"


def test_debug_quantize_cpu_matches_oracle(oracle):
    from bsipytorch_amd import bsi_ops

    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(500), [0.005, -0.005, 0.125, -2.675, 1e-7]]).astype(np.float32)
    for dec in (0, 2, 3):
        got = bsi_ops.debug_quantize_int64_cpu(torch.from_numpy(x), dec).numpy()
        np.testing.assert_array_equal(got, oracle.round_to_int64(x, dec))


def test_slice_weights_host(oracle):
    from bsipytorch_amd import bsi_ops

    for S, off, twos in [(7, 0, True), (6, 0, True), (4, 0, False), (3, 2, True)]:
        got = bsi_ops._slice_weights(S, off, twos, "cpu").numpy()
        np.testing.assert_array_equal(got, oracle.slice_weights(S, off, twos))


def test_dot_error_paths_on_host():
    from bsipytorch_amd import bsi_ops

    with pytest.raises(RuntimeError, match="Invalid CUDA keys capsule"):
        bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(object(), object())
    keys = bsi_ops.PrebuiltBSIKeysCUDA()
    with pytest.raises(RuntimeError, match="Invalid CUDA query-batch capsule"):
        bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(bsi_ops.PrebuiltBSIQueryCUDA(), keys)
    qb = bsi_ops.PrebuiltBSIQueryBatchCUDA()
    with pytest.raises(RuntimeError, match="not defined"):
        bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(qb, keys)
    qb.words = torch.zeros(2, 7, 4, dtype=torch.int64)
    qb.slice_weights = torch.zeros(2, 7)
    with pytest.raises(RuntimeError, match="must be CUDA tensors"):
        bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(qb, keys)
    with pytest.raises(RuntimeError, match="Empty keys or queries"):
        bsi_ops.batch_dot_product_multiquery_cuda_caps([], keys)
    with pytest.raises(RuntimeError, match="2D"):
        bsi_ops.build_bsi_queries_cuda_batch_packed(torch.zeros(4), 2)
    with pytest.raises(RuntimeError, match="2D"):
        bsi_ops.build_bsi_keys_cuda(torch.zeros(4), 2)
    with pytest.raises(RuntimeError, match="1D"):
        bsi_ops.build_bsi_query_cuda(torch.zeros(4, 4), 2)


def test_key_operand_selection_and_new_flags(monkeypatch):
    """Which key representation a dot reads: packed planes for a few query rows or the popcount core, the cached
    int8 image otherwise (host logic only: the tensors are never touched)."""
    from bsipytorch_amd import _lib, bsi_ops

    for k in list(os.environ):
        if k.startswith("BSI_"):
            monkeypatch.delenv(k)
    bsi_ops._reset_flag_cache()
    f = bsi_ops._flags()
    assert f["key_image"] and f["ewah_inline"]
    keys = bsi_ops.PrebuiltBSIKeysCUDA()
    keys.words = torch.zeros(4, dtype=torch.int64)
    keys.layout = _lib.LAYOUT_TILED16
    keys.ints8 = torch.zeros(16, dtype=torch.int8)
    planes = (keys.words.data_ptr(), _lib.LAYOUT_TILED16)
    image = (keys.ints8.data_ptr(), _lib.LAYOUT_INT8)
    assert bsi_ops.key_operand(keys, 1, 7, _lib.CORE_AUTO) == planes
    assert bsi_ops.key_operand(keys, 32, 7, _lib.CORE_MFMA) == planes
    assert bsi_ops.key_operand(keys, 33, 7, _lib.CORE_AUTO) == image
    assert bsi_ops.key_operand(keys, 512, 7, _lib.CORE_VALU) == planes      # the popcount core reads planes
    assert bsi_ops.key_operand(keys, 512, 12, _lib.CORE_AUTO) == planes     # values wider than int8
    keys.ints8 = None
    assert bsi_ops.key_operand(keys, 512, 7, _lib.CORE_AUTO) == planes
    monkeypatch.setenv("BSI_KEY_INT8_IMAGE", "0")
    monkeypatch.setenv("BSI_EWAH_INLINE", "0")
    bsi_ops._reset_flag_cache()
    f = bsi_ops._flags()
    assert not f["key_image"] and not f["ewah_inline"]
    bsi_ops._reset_flag_cache()


def test_set_option_validates_on_host():
    from bsipytorch_amd import _lib

    assert _lib.lib.bsi_hip_set_option(_lib.OPT_I8_TILE, 12864) == 0
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_I8_TILE, 6432) == 0
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_I8_TILE, 96) == 1
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_I8_TILE, 0) == 0
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_DIGITS_ROUTE, 2) == 0
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_DIGITS_ROUTE, 3) == 1
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_DIGITS_ROUTE, 0) == 0
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_BUILD_ITEMS, 4) == 0
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_BUILD_ITEMS, 3) == 1
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_BUILD_ITEMS, 0) == 0
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_I8_SPLIT, 6) == 0
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_I8_SPLIT, 65) == 1
    assert _lib.lib.bsi_hip_set_option(_lib.OPT_I8_SPLIT, 0) == 0
    assert _lib.lib.bsi_hip_set_option(999, 1) == 1
    assert b"unknown option" in _lib.lib.bsi_hip_last_error()


def test_split_scratch_host_side():
    """What the D-split's host side decides without touching a device: the scratch size that serves every choice, the
    refusal of a misaligned or too small region, detaching, and the plan of a thread with no region attached (the
    unsplit tile the launcher would take)."""
    import ctypes

    from bsipytorch_amd import _lib

    L = _lib.lib
    assert L.bsi_hip_dot_split_scratch_bytes() == 4096 + 256 * 128 * 128 * 4
    assert L.bsi_hip_dot_attach_split_scratch(None, 0) == 0                       # detaching is always fine
    assert L.bsi_hip_dot_attach_split_scratch(0x1008, 1 << 20) == 1 and b"aligned" in L.bsi_hip_last_error()
    assert L.bsi_hip_dot_attach_split_scratch(0x1000, 4096) == 1 and b"counters" in L.bsi_hip_last_error()
    tile, seg = ctypes.c_int(0), ctypes.c_int(0)
    for (R, Q, W), want in (((2048, 512, 128), 64), ((8192, 512, 32), 128), ((4096, 512, 64), 12864), ((4096, 128, 256), 6432)):
        assert L.bsi_hip_dot_split_plan(R, Q, W, ctypes.byref(tile), ctypes.byref(seg)) == 0
        assert (tile.value, seg.value) == (want, 1)
    assert L.bsi_hip_dot_split_plan(0, 512, 32, ctypes.byref(tile), ctypes.byref(seg)) == 1


def test_load_keyset_refuses_foreign_files_before_touching_the_device(tmp_path):
    from bsipytorch_amd import bsi_ops

    (tmp_path / "keyset.bsik").write_bytes(b"something else entirely")
    with pytest.raises(RuntimeError, match="not a BSI keyset file"):
        bsi_ops.load_keyset_cuda(str(tmp_path))
    (tmp_path / "keyset.bsik").write_bytes(b"BSIKEYS1" + (1 << 40).to_bytes(8, "little"))
    with pytest.raises(RuntimeError, match="bad header length"):
        bsi_ops.load_keyset_cuda(str(tmp_path))


def test_linear_few_rows_upfront_is_a_host_side_query():
    """bsi_hip_linear_few_rows_upfront needs no GPU: decode shapes of an OPT-6.7B layer at one row are served
    entirely up front, four rows of 16384 elements are not, bad shapes say no."""
    from bsipytorch_amd import _lib

    f = _lib.lib.bsi_hip_linear_few_rows_upfront
    assert f(1, 4096, 16384) == 1 and f(1, 16384, 4096) == 1 and f(1, 4096, 4096) == 1 and f(1, 4096, 12288) == 1
    assert f(4, 16384, 4096) == 0 and f(4, 4096, 16384) == 0
    assert f(2, 4096, 4096) == 1
    assert f(0, 4096, 4096) == 0 and f(5, 4096, 4096) == 0 and f(1, 0, 4096) == 0



def test_loader_raises_when_the_library_is_missing(monkeypatch, tmp_path):
    """Without libbsi_hip.so the package does not import: no CPU or PyTorch path stands in for the kernels."""
    from bsipytorch_amd import _lib

    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libbsi_hip.so"))
    with pytest.raises(ImportError, match="no fallback"):
        _lib._load()


def test_product_sources_never_reach_for_the_checker():
    """The CPU restatement under oracle/ is test infrastructure: no source of the package, the root `bsi_ops`
    shim or the C-ABI sources imports, links or names it (bench.py's CPU-baseline leg and smoke() are the only
    users outside tests/)."""
    offenders = []
    roots = [os.path.join(ROOT, "bsipytorch_amd"), os.path.join(ROOT, "include")]
    files = [os.path.join(ROOT, "bsi_ops.py")]
    for root in roots:
        for d, _, names in os.walk(root):
            files += [os.path.join(d, n) for n in names if n.endswith((".py", ".hip", ".h", ".cpp", ".c")) or n == "Makefile"]
    for f in files:
        if re.search(r"\boracle\b", open(f, errors="replace").read()):
            offenders.append(os.path.relpath(f, ROOT))
    assert offenders == []


# The launchers the reference's C++ declares (bsi_cuda.cpp:29-57, bsi_vector_cuda.cpp:91-242).
REFERENCE_LAUNCHERS = [
    "launch_ewah_decompress", "launch_popcount_weighted_keys_literal_fused_multiq", "launch_pack_bits_all_ballot",
    "launch_pack_bits_all_ballot_batch", "launch_quantize_round_to_int64_batch", "launch_compute_row_shift_scale",
    "launch_compute_chunk_shift_scale", "launch_apply_row_shift_clamp", "launch_apply_chunk_shift_clamp",
    "launch_compute_row_shift_scale_from_input", "launch_compute_chunk_shift_scale_from_input",
    "launch_quantize_shift_pack_row_batch", "launch_quantize_shift_pack_chunk_batch", "launch_slice_popcount_sum",
    "launch_compress_flags_from_density", "launch_ewah_size", "launch_ewah_emit",
]


def test_reference_launcher_library_exports_the_reference_symbols():
    """libbsi_reference_launchers.so (what a ROCm build of the reference extension links instead of its CUDA
    kernels) loads next to libbsi_hip.so and exports every launcher the reference's sources call."""
    path = os.path.join(ROOT, "bsipytorch_amd", "libbsi_reference_launchers.so")
    assert os.path.exists(path), "build it with make -C bsipytorch_amd/csrc"
    raw = ctypes.CDLL(path)
    for n in REFERENCE_LAUNCHERS:
        assert hasattr(raw, n), f"{n} is not exported"
    raw.bsi_launchers_last_error.restype = ctypes.c_char_p
    raw.bsi_launchers_clear_status()
    assert raw.bsi_launchers_last_status() == 0 and raw.bsi_launchers_last_error() == b""


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it exits with a message instead of a figure (no GPU needed to say so)."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    run = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)
    assert run.returncode == 2
    assert "one GPU" in run.stderr and not run.stdout.strip()
