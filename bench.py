"""Benchmark of the BSI fixed76 chunk-scale dot on one MI355X.

    python bench.py [--gpus 1] [--steps 50] [--warmup 10] [--settle-ms 60] [--core auto|mfma|valu] [--no-cpu] [--no-extras]

Workload: the FC1-like configuration (queries fp32 Q=512 x D=2048 ~N(0,1) with 0.1% of the columns
scaled x20, keys fp32 R=8192 x D=2048 ~N(0,0.02), decimal_places=2, compress_threshold=0.5, Sa=7,
Sb=6, chunk scales), synthetic, seed 123.  A step is one dot over the prebuilt query and key planes
(resident in HBM).  The headline (`value`, `ms_per_step`, `roofline`) is the W warm-up + K timed steps from an idle
GPU, the protocol of the reference's microbenchmark; "sustained" gives the same W + K steps after --settle-ms of
untimed steps, on the shader clock the GPU holds under load.
Prints ONE JSON line.  Its headline fields describe that workload; "other_configs" in the same line carries the
other benchmark configurations, each bounded to a few seconds: the correctness-scale shape, the FC2-like dot (with its
own roofline object, and with the queries kept as EWAH streams), the headline shape through the reference's own
launcher symbol, the OPT-6.7B layer shapes at 1, 16, 128 and 512 query rows (GB/s on the packed key planes, fraction
of the int8 peak), and the OPT-1.3B-shaped prefill (tokens/s eager and as a replayed HIP graph, share of the dot).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
MFMA_I8_PEAK_TOPS = 5000.0     # MI355X published dense int8
Q, R, D = 512, 8192, 2048
# HBM bytes per launch of the dot kernel on this workload: an OFFLINE figure, from rocprofv3 FETCH_SIZE and WRITE_SIZE
# runs of this script scaled by a 256 MiB copy (profiles/dot_mfma_i8_kernel_fc1_Q512_R8192_D2048_hbm_traffic.txt).
# Hardware counters cannot be read from inside the process, so it is not re-measured by a run of this script.
MEASURED_TRAFFIC_BYTES = {"mfma": 42439000}
TRAFFIC_SOURCE = "offline, profiles/..hbm_traffic.txt"
SA, SB = 7, 6


def _graph_timed_us(launches, rounds=4, replays=5):
    """Mean microseconds per launch of `launches` (callables that enqueue their kernels on the stream that is current
    when they are called: a capture makes its own stream current),
    recorded `rounds` times over into one HIP graph and replayed: no host work between the kernels, the same
    back-to-back conditions for one resident keyset and for a rotation of many."""
    import torch

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for f in launches:
            f()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(rounds):
            for f in launches:
                f()
    g.replay()
    torch.cuda.synchronize()
    best = None
    for _ in range(replays):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (rounds * len(launches))
        best = us if best is None else min(best, us)
    return best


def _idle_and_sustained_us(_lib, dot_args, iters, settle_ms, warmup=10):
    """(us per call from an idle GPU: `warmup` + `iters` back-to-back launches after a pause; us per call of `iters`
    launches after settle_ms of untimed ones, None when settle_ms is 0), by HIP events on the launch stream."""
    import torch

    st = torch.cuda.current_stream().cuda_stream
    us = ctypes.c_float(0.0)
    torch.cuda.synchronize()
    time.sleep(0.3)
    _lib.check(_lib.lib.bsi_hip_dot_timed(*dot_args, warmup, ctypes.byref(us), st), "warmup")
    _lib.check(_lib.lib.bsi_hip_dot_timed(*dot_args, iters, ctypes.byref(us), st), "timed")
    idle = float(us.value)
    if settle_ms <= 0:
        return idle, None
    _lib.check(_lib.lib.bsi_hip_dot_timed(*dot_args, max(1, int(settle_ms * 1e3 / idle)), ctypes.byref(us), st), "settle")
    _lib.check(_lib.lib.bsi_hip_dot_timed(*dot_args, iters, ctypes.byref(us), st), "timed")
    return idle, float(us.value)


def _compact(o):
    """Floats to five significant digits: the line stays short enough for whatever keeps only the end of the output."""
    if isinstance(o, float):
        return float(f"{o:.5g}")
    if isinstance(o, dict):
        return {k: _compact(v) for k, v in o.items()}
    if isinstance(o, (list, tuple)):
        return [_compact(v) for v in o]
    return o


def _fc2_like(_lib, bsi_ops, iters, settle_ms):
    """FC2-like dot Q512 x R2048 x D8192, ReLU queries: the int8-image kernel on the verbatim batch, and the same
    batch kept as EWAH streams (decode launch + dot) next to the verbatim planes taken through the same two steps."""
    import torch

    Q3, R3, D3 = 512, 2048, 8192
    torch.manual_seed(123)
    X = torch.relu(torch.randn(Q3, D3))
    K = torch.randn(R3, D3) * 0.02
    kcap, _, _, _, W = bsi_ops.build_bsi_keys_cuda(K, 2, 0.5)
    qcap = bsi_ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.5)
    hb = bsi_ops.build_bsi_queries_cuda_batch_hybrid(X.cuda(), 2, 0.5)
    chunks = W // 4
    out = torch.empty((Q3, R3), dtype=torch.float32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    kptr, klayout = bsi_ops.key_operand(kcap, Q3, SA, _lib.CORE_MFMA)
    us = ctypes.c_float(0.0)
    args = (qcap.words.data_ptr(), qcap.ints8.data_ptr(), qcap.chunk_scales.data_ptr(), chunks, SA, W, kptr, klayout,
            kcap.slice_weights.data_ptr(), SB, R3, Q3, 1e-4, R3, out.data_ptr(), _lib.CORE_MFMA, None, 0)
    first_us, settled_us = _idle_and_sustained_us(_lib, args, iters, settle_ms)
    int8_ops = 2.0 * Q3 * R3 * D3
    alg_bytes = Q3 * SA * W * 8 + Q3 * chunks * 4 + R3 * SB * W * 8 + R3 * 4 + Q3 * R3 * 4
    t_idle = first_us * 1e-6
    # both published roofs lie far below this launch (3.44 us of int8 MFMA, 2.57 us of HBM on the algorithmic bytes);
    # the larger floor is the int8 one here, so that is the roofline object; the HBM fraction stands beside it
    res = {"workload": "FC2-like dot Q512 R2048 D8192, ReLU queries", "us_per_call": first_us,
           "effective_bitop_TOPS": 2.0 * SA * SB * Q3 * R3 * D3 / t_idle / 1e12,
           "roofline": {"bound": "mfma", "achieved": int8_ops / t_idle / 1e12, "peak": MFMA_I8_PEAK_TOPS, "unit": "TOP/s",
                        "frac": int8_ops / t_idle / 1e12 / MFMA_I8_PEAK_TOPS, "traffic": None,
                        "frac_of_hbm_peak_algorithmic": alg_bytes / t_idle / 1e9 / HBM_PEAK_GBS},
           "us_per_call_sustained": settled_us}
    # queries as EWAH streams: the dot's load stage turns the streams into the int8 image (one launch), then the same
    # kernel runs; next to it the verbatim planes through planes -> int8 image -> dot (what a caller holding planes pays)
    ws_bytes = int(_lib.lib.bsi_hip_dot_ewah_batch_workspace_bytes(Q3, W))
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device="cuda")

    def ewah():
        _lib.check(_lib.lib.bsi_hip_dot_ewah_batch(hb.comp_words.data_ptr(), hb.comp_off.data_ptr(), hb.comp_len.data_ptr(),
                                                   SA, W, hb.chunk_scales.data_ptr(), chunks, kptr, klayout,
                                                   kcap.slice_weights.data_ptr(), SB, R3, Q3, 1e-4, R3, None, out.data_ptr(),
                                                   None, ws.data_ptr(), ws_bytes, bsi_ops._stream()), "bsi_hip_dot_ewah_batch")

    def planes():
        _lib.check(_lib.lib.bsi_hip_dot(qcap.words.data_ptr(), None, qcap.chunk_scales.data_ptr(), chunks, SA, W, kptr,
                                        klayout, kcap.slice_weights.data_ptr(), SB, R3, Q3, 1e-4, R3, out.data_ptr(), None,
                                        _lib.CORE_MFMA, ws.data_ptr(), ws_bytes, bsi_ops._stream()), "bsi_hip_dot")

    res["ewah_queries"] = {
        "us_per_call_streams": _graph_timed_us([ewah], rounds=8) ,
        "us_per_call_verbatim_planes": _graph_timed_us([planes], rounds=8),
        "stored_query_bytes_streams": int(hb.mem_bytes), "stored_query_bytes_verbatim": int(hb.verbatim_bytes)}
    # a few rows (16 tokens against an OPT-6.7B attention projection): the streams are expanded inside the dot kernel
    R6 = D6 = 4096
    g6 = torch.Generator(device="cuda").manual_seed(6)
    k6 = bsi_ops.build_bsi_keys_cuda(torch.randn(R6, D6, device="cuda", generator=g6) * 0.02, 2, 0.5)[0]
    x6 = torch.relu(torch.randn(16, D6, device="cuda", generator=g6))
    q6, h6 = bsi_ops.build_bsi_queries_cuda_batch_packed(x6, 2, 0.5), bsi_ops.build_bsi_queries_cuda_batch_hybrid(x6, 2, 0.5)
    o6 = torch.empty((16, R6), dtype=torch.float32, device="cuda")

    def few_streams():
        _lib.check(_lib.lib.bsi_hip_dot_ewah_batch(h6.comp_words.data_ptr(), h6.comp_off.data_ptr(), h6.comp_len.data_ptr(), SA,
                                                   D6 // 64, h6.chunk_scales.data_ptr(), D6 // 256, k6.words.data_ptr(), k6.layout,
                                                   k6.slice_weights.data_ptr(), SB, R6, 16, 1e-4, R6, None, o6.data_ptr(), None,
                                                   None, 0, bsi_ops._stream()), "bsi_hip_dot_ewah_batch")

    def few_verbatim():
        _lib.check(_lib.lib.bsi_hip_dot(q6.words.data_ptr(), q6.ints8.data_ptr(), q6.chunk_scales.data_ptr(), D6 // 256, SA,
                                        D6 // 64, k6.words.data_ptr(), k6.layout, k6.slice_weights.data_ptr(), SB, R6, 16, 1e-4,
                                        R6, o6.data_ptr(), None, _lib.CORE_MFMA, None, 0, bsi_ops._stream()), "bsi_hip_dot")

    res["ewah_queries"]["few_rows_Q16_R4096_D4096"] = {"us_streams_decoded_in_kernel": _graph_timed_us([few_streams], rounds=16),
                                                       "us_verbatim_int8_image": _graph_timed_us([few_verbatim], rounds=16)}
    ewah()
    torch.cuda.synchronize()
    a = out.clone()
    planes()
    torch.cuda.synchronize()
    res["ewah_queries"]["bit_identical_to_verbatim"] = bool(torch.equal(a, out))
    return res


def _decode_shapes(_lib, bsi_ops):
    """OPT-6.7B layer shapes.  At ONE query row (the HBM-bound decode regime): microseconds and GB/s on the packed key
    planes (0.75 byte per weight), on one resident keyset and on a rotation of keysets larger than the 256 MB
    memory-side cache, so that every launch reads its planes from HBM.  At 16, 128 and 512 rows: microseconds on one
    resident keyset, with GB/s on the planes (16 rows) or the fraction of the int8 peak (128, 512 rows)."""
    import torch

    rows = []
    for name, R5, D5 in (("attn 4096x4096", 4096, 4096), ("fc1 16384x4096", 16384, 4096), ("fc2 4096x16384", 4096, 16384)):
        plane_bytes = R5 * SB * (D5 // 64) * 8
        n_sets = max(2, -(-640 * 1024 * 1024 // plane_bytes))           # at least 640 MB of planes in rotation
        gen = torch.Generator(device="cuda").manual_seed(R5 + D5)
        keysets = []
        for _ in range(n_sets):
            Kd = torch.randn(R5, D5, device="cuda", generator=gen) * 0.02
            keysets.append(bsi_ops.build_bsi_keys_cuda(Kd, 2, 0.5)[0])
            del Kd
        for kc in keysets:
            kc.ints8 = None                                            # the image is not read at one row: free it
        x = torch.randn(1, D5, device="cuda", generator=gen)
        qcap = bsi_ops.build_bsi_queries_cuda_batch_packed(x, 2, 0.5)
        W, chunks = D5 // 64, D5 // 256
        out = torch.empty((1, R5), dtype=torch.float32, device="cuda")

        def launch(kc):
            def f():
                _lib.check(_lib.lib.bsi_hip_dot(qcap.words.data_ptr(), qcap.ints8.data_ptr(), qcap.chunk_scales.data_ptr(),
                                                chunks, SA, W, kc.words.data_ptr(), kc.layout, kc.slice_weights.data_ptr(),
                                                SB, R5, 1, 1e-4, R5, out.data_ptr(), None, _lib.CORE_MFMA, None, 0, bsi_ops._stream()),
                           "bsi_hip_dot")
            return f

        resident = _graph_timed_us([launch(keysets[0])], rounds=32)
        rotating = _graph_timed_us([launch(kc) for kc in keysets], rounds=2)
        row = {"layer": name, "Q1_us": resident, "Q1_GBs_on_planes": plane_bytes / resident / 1e3,
               "Q1_us_rotating": rotating, "Q1_GBs_on_planes_rotating": plane_bytes / rotating / 1e3}
        # the same layer at 16, 128 and 512 rows (one resident keyset, from an idle GPU, 10 + 50 launches): GB/s on the
        # packed planes while the call is bandwidth-bound, fraction of the int8 peak where it is compute-bound
        kc = bsi_ops.build_bsi_keys_cuda(torch.randn(R5, D5, device="cuda", generator=gen) * 0.02, 2, 0.5)[0]
        del keysets
        torch.cuda.empty_cache()
        for Qn in (16, 128, 512):
            xq = torch.randn(Qn, D5, device="cuda", generator=gen)
            qc = bsi_ops.build_bsi_queries_cuda_batch_packed(xq, 2, 0.5)
            on = torch.empty((Qn, R5), dtype=torch.float32, device="cuda")
            kptr, klayout = bsi_ops.key_operand(kc, Qn, SA, _lib.CORE_MFMA)
            bsi_ops.attach_split_scratch()
            a = (qc.words.data_ptr(), qc.ints8.data_ptr(), qc.chunk_scales.data_ptr(), chunks, SA, W, kptr, klayout,
                 kc.slice_weights.data_ptr(), SB, R5, Qn, 1e-4, R5, on.data_ptr(), _lib.CORE_MFMA, None, 0)
            us_n, _ = _idle_and_sustained_us(_lib, a, 50, 0)
            row[f"Q{Qn}_us"] = us_n
            if Qn <= 32:
                row[f"Q{Qn}_GBs_on_planes"] = plane_bytes / us_n / 1e3
            else:
                row[f"Q{Qn}_frac_of_int8_peak"] = 2.0 * Qn * R5 * D5 / (us_n * 1e-6) / 1e12 / MFMA_I8_PEAK_TOPS
        rows.append(row)
        del kc
        torch.cuda.empty_cache()
    return rows


def _correctness_scale(_lib, bsi_ops):
    """The correctness-scale shape (Q64 R256 D2048, keys ~N(0, 0.02)): microseconds per call and the relative error
    against the dense fp32 product (the quantisation grid, not arithmetic error: the dot is exact on its integers)."""
    import torch

    torch.manual_seed(123)
    X, K = torch.randn(64, 2048), torch.randn(256, 2048) * 0.02
    kcap, _, _, _, W = bsi_ops.build_bsi_keys_cuda(K, 2, 0.5)
    qcap = bsi_ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.5)
    out = torch.empty((64, 256), dtype=torch.float32, device="cuda")
    kptr, klayout = bsi_ops.key_operand(kcap, 64, SA, _lib.CORE_MFMA)
    a = (qcap.words.data_ptr(), qcap.ints8.data_ptr(), qcap.chunk_scales.data_ptr(), W // 4, SA, W, kptr, klayout,
         kcap.slice_weights.data_ptr(), SB, 256, 64, 1e-4, 256, out.data_ptr(), _lib.CORE_MFMA, None, 0)
    us, _ = _idle_and_sustained_us(_lib, a, 50, 0)
    dense = X.double() @ K.double().T
    rel = float(torch.linalg.norm(out.cpu().double() - dense) / torch.linalg.norm(dense))
    return {"workload": "Q64 R256 D2048", "us_per_call": us, "rel_error_vs_dense_fp32": rel}


def _through_reference_launcher(_lib, bsi_ops, X, qcap, kcap_canonical, out_ref, iters):
    """The headline shape through launch_popcount_weighted_keys_literal_fused_multiq of libbsi_reference_launchers.so,
    the reference's own dot launcher symbol with its 19 arguments and canonical planes: as handed over (the
    plane-reading kernel), and with the keyset registered (bsi_launchers_register_keys: the int8 image route, the
    query planes packed through the reference's own builder launchers as bsi_vector_cuda.cpp:401-557 calls them)."""
    import torch

    vp, i32, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    L = ctypes.CDLL(os.path.join(ROOT, "bsipytorch_amd", "libbsi_reference_launchers.so"))
    L.launch_popcount_weighted_keys_literal_fused_multiq.argtypes = [vp, vp, vp, i32, i32, i32, vp, vp, i32, i32, i32, i32,
                                                                     i32, vp, vp, f32, i32, vp, vp]
    L.launch_popcount_weighted_keys_literal_fused_multiq.restype = None
    L.bsi_launchers_register_keys.argtypes, L.bsi_launchers_register_keys.restype = [vp, i32, i32, i32, vp], i32
    L.bsi_launchers_forget_keys.argtypes, L.bsi_launchers_forget_keys.restype = [vp], i32
    L.bsi_launchers_last_error.restype = ctypes.c_char_p
    i64, f64, u64 = ctypes.c_int64, ctypes.c_double, ctypes.c_uint64
    L.launch_compute_chunk_shift_scale_from_input.argtypes = [vp, i32, i64, i64, i32, f64, i32, f32, vp, vp, vp]
    L.launch_compute_chunk_shift_scale_from_input.restype = None
    L.launch_quantize_shift_pack_chunk_batch.argtypes = [vp, i32, i64, i64, i32, i32, i32, u64, f64, i32, vp, vp, vp]
    L.launch_quantize_shift_pack_chunk_batch.restype = None
    W, chunks = D // 64, D // 256
    out = torch.empty((Q, R), dtype=torch.float32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    words, scales = qcap.words, qcap.chunk_scales

    def launch():
        L.launch_popcount_weighted_keys_literal_fused_multiq(words.data_ptr(), qcap.slice_weights.data_ptr(),
                                                             scales.data_ptr(), chunks, SA, W,
                                                             kcap_canonical.words.data_ptr(), kcap_canonical.slice_weights.data_ptr(),
                                                             SB, R, Q, 8, 4, None, None, 1e-4, R, out.data_ptr(), st)

    def timed():
        for _ in range(10):
            launch()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        time.sleep(0.3)
        e0.record()
        for _ in range(iters):
            launch()
        e1.record()
        torch.cuda.synchronize()
        assert L.bsi_launchers_last_status() == 0, L.bsi_launchers_last_error()
        return e0.elapsed_time(e1) * 1e3 / iters

    res = {"us_planes_as_handed_over": timed()}
    assert L.bsi_launchers_register_keys(kcap_canonical.words.data_ptr(), R, SB, W, st) == 0
    xd = X.cuda()
    words, scales = torch.empty_like(qcap.words), torch.empty_like(qcap.chunk_scales)
    shifts = torch.empty((Q, chunks), dtype=torch.int32, device="cuda")
    L.launch_compute_chunk_shift_scale_from_input(xd.data_ptr(), 0, Q, D, chunks, 100.0, SA, 0.0, shifts.data_ptr(),
                                                  scales.data_ptr(), st)
    L.launch_quantize_shift_pack_chunk_batch(xd.data_ptr(), 0, Q, D, chunks, SA, W, (1 << SA) - 1, 100.0, SA, shifts.data_ptr(),
                                             words.data_ptr(), st)
    res["us_keys_registered"] = timed()
    res["bit_identical"] = bool(torch.equal(out, out_ref))
    L.bsi_launchers_forget_keys(kcap_canonical.words.data_ptr())
    return res


def _headline_rotating(_lib, bsi_ops):
    """The headline shape (Q512 R8192 D2048) on a rotation of keysets whose int8 images add up to more than the 256 MB
    memory-side cache, so that every launch reads its 16 MiB key image from HBM, next to the resident figure taken the
    same way (launches recorded into one HIP graph and replayed)."""
    import torch

    Qh, Rh, Dh = 512, 8192, 2048
    image_bytes = Rh * Dh
    n_sets = -(-640 * 1024 * 1024 // image_bytes)
    gen = torch.Generator(device="cuda").manual_seed(7)
    keysets = []
    for _ in range(n_sets):
        Kd = torch.randn(Rh, Dh, device="cuda", generator=gen) * 0.02
        keysets.append(bsi_ops.build_bsi_keys_cuda(Kd, 2, 0.5)[0])
        del Kd
    x = torch.randn(Qh, Dh, device="cuda", generator=gen)
    qcap = bsi_ops.build_bsi_queries_cuda_batch_packed(x, 2, 0.5)
    W, chunks = Dh // 64, Dh // 256
    out = torch.empty((Qh, Rh), dtype=torch.float32, device="cuda")

    def launch(kc):
        kptr, klayout = bsi_ops.key_operand(kc, Qh, SA, _lib.CORE_MFMA)

        def f():
            _lib.check(_lib.lib.bsi_hip_dot(qcap.words.data_ptr(), qcap.ints8.data_ptr(), qcap.chunk_scales.data_ptr(),
                                            chunks, SA, W, kptr, klayout, kc.slice_weights.data_ptr(), SB, Rh, Qh, 1e-4, Rh,
                                            out.data_ptr(), None, _lib.CORE_MFMA, None, 0, bsi_ops._stream()), "bsi_hip_dot")
        return f

    resident = _graph_timed_us([launch(keysets[0])], rounds=32)
    rotating = _graph_timed_us([launch(kc) for kc in keysets], rounds=2)
    ops = 2.0 * Qh * Rh * Dh
    return {"keysets_in_rotation": n_sets,
            "us_resident": resident, "us_rotating": rotating,
            "frac_of_int8_mfma_peak_rotating": ops / (rotating * 1e-6) / 1e12 / MFMA_I8_PEAK_TOPS}


def _opt_prefill():
    """OPT-1.3B-shaped prefill (24 layers, hidden 2048, 32 heads, FFN 8192, vocab 50272, batch 1 x 512 tokens, every
    decoder linear layer BSI): tokens/s eager and as a replayed HIP graph, and the dot's share of the forward."""
    from bsipytorch_amd.benchmarks import benchmark_opt_prefill

    r = benchmark_opt_prefill.run("opt-1.3b", seq_len=512, batch=1, iters=5, warmup=2, dense=False, graph=True)
    # dot_gpu_ms / query_build_gpu_ms: GPU time of those launches alone, replayed from a graph without
    # synchronisation; their shares are of the replayed forward
    keep = ("model", "seq_len", "num_bsi_layers", "bsi_fwd_ms", "bsi_tokens_per_s", "bsi_graph_fwd_ms",
            "bsi_graph_tokens_per_s", "graph_replays_match_eager", "dot_gpu_ms_per_prefill", "dot_share_of_graph_fwd",
            "query_build_gpu_ms_per_prefill", "query_build_share_of_graph_fwd")
    res = {k: r[k] for k in keep if k in r}
    # the same model with q_proj, k_proj and v_proj of every layer served by one dot (same bits, one launch for three)
    f = benchmark_opt_prefill.run("opt-1.3b", seq_len=512, batch=1, iters=5, warmup=2, dense=False, graph=True,
                                  fuse_qkv=True)
    res["one_dot_for_q_k_v"] = {k: f[k] for k in ("bsi_fwd_ms", "bsi_tokens_per_s", "bsi_graph_fwd_ms",
                                                   "bsi_graph_tokens_per_s", "graph_replays_match_eager") if k in f}
    return res


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--core", default="auto", choices=["auto", "mfma", "valu"])
    ap.add_argument("--settle-ms", type=float, default=60.0,
                    help="the W + K steps are timed twice: from an idle GPU (the headline) and behind this many "
                         "milliseconds of untimed back-to-back steps (\"sustained\": the shader clock the GPU holds under "
                         "load, which power management reaches after about 35 ms); 0 = from idle only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip the other configurations (FC2-like, decode shapes, prefill)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a dispatch of known traffic for scaling "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no collectives); run with --gpus 1",
              file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from bsipytorch_amd import _lib, bsi_ops

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)
    torch.manual_seed(123)
    X = torch.randn(Q, D)
    cols = torch.randperm(D)[: max(1, D // 1000)]
    X[:, cols] *= 20.0
    K = torch.randn(R, D) * 0.02

    kcap, _, _, _, W = bsi_ops.build_bsi_keys_cuda(K, 2, 0.5)
    qcap = bsi_ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.5)
    chunks = W // 4
    core = {"auto": _lib.CORE_AUTO, "mfma": _lib.CORE_MFMA, "valu": _lib.CORE_VALU}[args.core]
    out = torch.empty((Q, R), dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    scale_inv = 1.0 / 10.0 ** 4

    kptr, klayout = bsi_ops.key_operand(kcap, Q, SA, core)

    def dot_args():
        return (qcap.words.data_ptr(), qcap.ints8.data_ptr(), qcap.chunk_scales.data_ptr(), chunks, SA, W,
                kptr, klayout, kcap.slice_weights.data_ptr(), SB, R, Q, scale_inv, R, out.data_ptr())

    def step():
        _lib.check(_lib.lib.bsi_hip_dot(*dot_args(), None, core, None, 0, stream), "bsi_hip_dot")

    if args.calibration_copy:
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def timed_steps():
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps

    # The headline is the reference microbenchmark's protocol: W warm-up + K timed steps from an idle GPU.  The shader
    # clock is regulated over tens of milliseconds (a call takes 13.5 - 15 us during the first milliseconds of load and
    # settles about 10 % lower after some 35 ms), so the same W + K steps are timed again behind --settle-ms of untimed
    # steps and reported as "sustained", with fractions of their own: what a serving loop sees.
    mean_us = ctypes.c_float(0.0)

    def kernel_us():  # HIP events on the launch stream around W, then K back-to-back launches
        _lib.check(_lib.lib.bsi_hip_dot_timed(*dot_args(), core, None, 0, max(1, args.warmup), ctypes.byref(mean_us), stream), "warmup")
        _lib.check(_lib.lib.bsi_hip_dot_timed(*dot_args(), core, None, 0, args.steps, ctypes.byref(mean_us), stream), "bsi_hip_dot_timed")
        return float(mean_us.value)

    torch.cuda.synchronize()
    time.sleep(0.3)
    ms_per_step = timed_steps()
    torch.cuda.synchronize()
    time.sleep(0.3)
    kern_us = kernel_us()
    sustained = None
    if args.settle_ms > 0:
        settle_steps = max(1, int(args.settle_ms / ms_per_step))
        for _ in range(settle_steps):  # no synchronisation in between: an idle gap would let the clock state decay
            step()
        sustained_ms = timed_steps()
        _lib.check(_lib.lib.bsi_hip_dot_timed(*dot_args(), core, None, 0, settle_steps, ctypes.byref(mean_us), stream), "settle")
        sustained = {"settle_ms": args.settle_ms, "untimed_steps": settle_steps, "us_per_call": sustained_ms * 1e3,
                     "kernel_us": kernel_us()}

    bit_ops = 2.0 * SA * SB * Q * R * D                  # one AND + one popcount-accumulate per bit-MAC
    int8_ops = 2.0 * Q * R * D                           # the same contraction counted as int8 MACs
    alg_bytes = Q * SA * W * 8 + Q * chunks * 4 + R * SB * W * 8 + R * 4 + Q * R * 4
    used_core = args.core if args.core != "auto" else "mfma"
    hbm_gbs = alg_bytes / (kern_us * 1e-6) / 1e9
    if used_core == "mfma":
        # Two published roofs apply to the int8 MFMA contraction of this shape and lie close together: 2*Q*R*D int8
        # operations against the dense int8 peak (floor 3.44 us) and the algorithmic bytes against HBM (floor 3.79 us).
        # The larger floor binds, so the roofline object is the HBM one; both fractions are reported.
        mfma_tops = int8_ops / (kern_us * 1e-6) / 1e12
        floors = {"mfma_us": int8_ops / (MFMA_I8_PEAK_TOPS * 1e12) * 1e6, "hbm_us": alg_bytes / (HBM_PEAK_GBS * 1e9) * 1e6}
        roof = {"bound": "hbm", "achieved": hbm_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "floors_us": floors,
                "mfma": {"achieved": mfma_tops, "peak": MFMA_I8_PEAK_TOPS, "unit": "TOP/s",
                         "frac": mfma_tops / MFMA_I8_PEAK_TOPS}}
    else:
        # The popcount core is VALU-bound, which the two published roofs do not describe; it is priced
        # against HBM here and against the VALU issue rate in "valu" below.
        roof = {"bound": "hbm", "achieved": hbm_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = MEASURED_TRAFFIC_BYTES.get(used_core)
    roof["traffic_source"] = TRAFFIC_SOURCE if roof["traffic"] is not None else None
    roof["kernel_us"] = kern_us
    # one v_and_b32 + one v_bcnt_u32_b32 per 32 bit-MACs; 256 CU x 4 SIMD x 16 lanes x 2.4 GHz lane-ops/s
    valu_peak = 256 * 4 * 16 * 2.4e9 * 32 / 2 / 1e12
    valu = {"achieved_Tbitmac_s": bit_ops / 2 / (kern_us * 1e-6) / 1e12, "peak_Tbitmac_s": valu_peak}
    valu["frac"] = valu["achieved_Tbitmac_s"] / valu_peak

    result = {
        "metric": "bsi_dot_effective_bitop_TOPS@Q512_R8192_D2048",
        "value": bit_ops / (ms_per_step * 1e-3) / 1e12,
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8" if used_core == "mfma" else "u32",
        "data": "synthetic",
        "config": {"workload": "FC1-like fixed76 chunk-scale dot Q512 R8192 D2048, 0.1% outlier columns x20, dec=2",
                   "core": used_core, "protocol": "W + K steps from an idle GPU", "algorithmic_bytes": alg_bytes},
        "roofline": roof,
    }
    if sustained is not None:
        ks = sustained["kernel_us"] * 1e-6
        sustained["value"] = bit_ops / (sustained["us_per_call"] * 1e-6) / 1e12
        sustained["frac_of_hbm_peak"] = alg_bytes / ks / 1e9 / HBM_PEAK_GBS
        sustained["frac_of_int8_mfma_peak"] = int8_ops / ks / 1e12 / MFMA_I8_PEAK_TOPS
        result["sustained"] = sustained
    if used_core == "valu":
        result["valu"] = valu

    # peaks measured on this GPU by the library's probes (a pure v_mfma_i32_16x16x64_i8 loop, a pure
    # v_and/v_bcnt loop, a streaming read of 1 GiB), next to the published figures the roofline uses
    peaks = {}
    v = ctypes.c_double(0.0)
    _lib.check(_lib.lib.bsi_hip_probe_mfma_i8(ctypes.byref(v), stream), "probe_mfma")
    peaks["int8_mfma_TOPS"] = v.value / 1e12
    # the same loop on pseudo-random bytes shaped like the dot's images: the clock follows the data's switching
    # activity, so this is the rate real operands can sustain on the matrix pipes alone
    _lib.check(_lib.lib.bsi_hip_probe_mfma_i8_operands(1, ctypes.byref(v), stream), "probe_mfma_operands")
    peaks["int8_mfma_TOPS_random_operands"] = v.value / 1e12
    _lib.check(_lib.lib.bsi_hip_probe_valu_popcount(ctypes.byref(v), stream), "probe_valu")
    peaks["valu_and_bcnt_Tbitmac_s"] = v.value * 32 / 2 / 1e12   # one v_and + one v_bcnt per 32 bit-MACs
    buf = torch.ones(1 << 30, dtype=torch.uint8, device="cuda")
    _lib.check(_lib.lib.bsi_hip_probe_stream_read(buf.data_ptr(), buf.numel(), ctypes.byref(v), stream), "probe_read")
    peaks["stream_read_GBs"] = v.value / 1e9
    # the int8-image kernel's operand path: L2-resident bytes into LDS by LDS-direct loads, every CU at once -- with
    # eight issuing waves and contiguous pieces (the path's best), and as the kernel's four loader waves issue them
    _lib.check(_lib.lib.bsi_hip_probe_l2_to_lds(buf.data_ptr(), buf.numel(), 0, ctypes.byref(v), stream), "probe_l2_lds")
    peaks["l2_to_lds_GBs"] = v.value / 1e9
    _lib.check(_lib.lib.bsi_hip_probe_l2_to_lds(buf.data_ptr(), buf.numel(), 1, ctypes.byref(v), stream), "probe_l2_lds")
    peaks["l2_to_lds_GBs_four_loader_waves_row_pieces"] = v.value / 1e9
    del buf
    result["measured_peaks"] = peaks
    result["roofline"]["frac_of_measured_mfma_peak"] = (int8_ops / (kern_us * 1e-6) / 1e12) / peaks["int8_mfma_TOPS"]

    # dense baselines of the same shape on the same GPU (resident operands, same event timing)
    Xd, Kd = X.cuda(), K.cuda()
    dense = {}
    for name, dt in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
        a, b = Xd.to(dt), Kd.to(dt)
        for _ in range(5):
            torch.matmul(a, b.T)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            torch.matmul(a, b.T)
        e1.record()
        torch.cuda.synchronize()
        dense[f"torch_matmul_{name}_us"] = e0.elapsed_time(e1) / 20 * 1e3
    # the vendor library's int8 GEMM of the shape (int32 output, no chunk scales): the same matrix-core instruction
    # class as the BSI dot's core, without its fp32 chain
    try:
        a8 = torch.randint(-64, 63, (Q, D), dtype=torch.int8, device="cuda")
        b8 = torch.randint(-32, 31, (R, D), dtype=torch.int8, device="cuda")
        for _ in range(5):
            torch._int_mm(a8, b8.t())
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            torch._int_mm(a8, b8.t())
        e1.record()
        torch.cuda.synchronize()
        dense["torch_int_mm_int8_us"] = e0.elapsed_time(e1) / 20 * 1e3
    except Exception as exc:  # not every build of torch has it
        dense["torch_int_mm_int8_us"] = None
        dense["torch_int_mm_error"] = f"{type(exc).__name__}: {exc}"[:200]
    result["dense_baseline"] = dense

    if not args.no_cpu:
        from oracle import bsi_oracle

        A = qcap.words.cpu().numpy().view(np.uint64)
        qs = qcap.chunk_scales.cpu().numpy()
        # canonical key planes for the oracle (rebuilt on the GPU in canonical order, then copied)
        os.environ["BSI_KEY_LAYOUT"] = "canonical"
        bsi_ops._reset_flag_cache()
        kc, *_ = bsi_ops.build_bsi_keys_cuda(K, 2, 0.5)
        del os.environ["BSI_KEY_LAYOUT"]
        bsi_ops._reset_flag_cache()
        B = kc.words.cpu().numpy().view(np.uint64)
        bs = kc.slice_weights[:, 0].contiguous().cpu().numpy()
        reps, t_cpu = 0, 0.0
        while t_cpu < 12.0 and reps < 100:  # a bounded sample: about 12 s of CPU work, whole passes only
            t1 = time.perf_counter()
            _, ref = bsi_oracle.dot_fixed(A, qs, B, bs, np.float32(scale_inv), want_ints=False)
            t_cpu += time.perf_counter() - t1
            reps += 1
        step()
        torch.cuda.synchronize()
        same = bool(np.array_equal(out.cpu().numpy(), ref))
        result["cpu_baseline"] = {"value": bit_ops / (t_cpu / reps) / 1e12, "unit": "TOPS", "cores": bsi_oracle.num_threads(),
                                  "kind": "port", "sample": f"{reps} full passes of the same dot",
                                  "ms_per_call": t_cpu / reps * 1e3, "gpu_output_bit_identical": same}
    if not args.no_extras and used_core == "mfma":
        extras = {}
        def launcher_leg():
            os.environ["BSI_KEY_LAYOUT"] = "canonical"
            bsi_ops._reset_flag_cache()
            try:
                kc_canonical = bsi_ops.build_bsi_keys_cuda(K, 2, 0.5)[0]
            finally:
                del os.environ["BSI_KEY_LAYOUT"]
                bsi_ops._reset_flag_cache()
            step()
            torch.cuda.synchronize()
            return _through_reference_launcher(_lib, bsi_ops, X, qcap, kc_canonical, out, args.steps)

        for key, fn in (("c1_correctness_scale", lambda: _correctness_scale(_lib, bsi_ops)),
                        ("fc2_like", lambda: _fc2_like(_lib, bsi_ops, args.steps, args.settle_ms)),
                        ("headline_through_reference_launcher", launcher_leg),
                        ("headline_on_rotating_keysets", lambda: _headline_rotating(_lib, bsi_ops)),
                        ("opt6.7b_layers", lambda: _decode_shapes(_lib, bsi_ops)),
                        ("opt1.3b_prefill", _opt_prefill)):
            try:
                extras[key] = fn()
            except Exception as exc:  # the headline line must not be lost to a side figure
                extras[key] = {"error": f"{type(exc).__name__}: {exc}"}
            torch.cuda.empty_cache()
        result["other_configs"] = extras
    print(json.dumps(_compact(result)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
