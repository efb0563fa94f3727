"""The reference's scalar ("non-CUDA") ``bsi_ops`` entry points (bsiFunctions.cpp:811-846), served by the device kernels.

In the reference these functions build bsiCPP ``BsiVector`` objects on the host and call ``BsiVector::dot``; the
bsiCPP library is not part of the reference's tree.  What the functions compute is fixed by their own source
all the same: the integers come from a stated rule (``static_cast<long>(x * factor)`` or round half away of
``x * 10^dec``), ``dot`` of two bit-sliced vectors is the exact integer dot product of those integers, and the
result is that integer divided by a stated scale.  Here the integers are produced by the device quantisers, sliced
by the decimal-mode builder and contracted by the weighted-slice dot kernel in float64 (exact below 2^53), so the
values are the reference's.  The byte counts and slice statistics describe THIS build's slices (two's-complement
planes with the decimal builder's slice count; EWAH streams where the density flag says so) -- bsiCPP's own slice
rule and container sizes are not recoverable from the reference's tree, and nothing can pin those numbers.

Every function needs the HIP library and a GPU, like the rest of the module; inputs may live on either device and
results come back where the reference returns them (Python numbers, CPU tensors).
"""
import os
from typing import Tuple

import numpy as np
import torch

from . import _lib
from ._lib import check, lib


def _ops():
    from . import bsi_ops

    return bsi_ops


def _vec(t: torch.Tensor, what: str) -> torch.Tensor:
    ops = _ops()
    ops._check(isinstance(t, torch.Tensor) and t.dim() == 1, f"{what} must be 1D")
    return t.detach().to(device=ops._device(), dtype=torch.float32).contiguous()


def _mat(t: torch.Tensor, what: str) -> torch.Tensor:
    ops = _ops()
    ops._check(isinstance(t, torch.Tensor) and t.dim() == 2, f"{what} must be 2D")
    return t.detach().to(device=ops._device(), dtype=torch.float32).contiguous()


def _ints_trunc(x2d: torch.Tensor, factor: float) -> torch.Tensor:
    """(int64)(x * factor), product in float32, conversion towards zero (bsiFunctions.cpp:265-271)."""
    out = torch.empty(x2d.shape, dtype=torch.int64, device=x2d.device)
    if x2d.numel():
        check(lib.bsi_hip_quantize_trunc_to_int64(x2d.data_ptr(), _lib.DTYPE_F32, x2d.numel(), float(factor),
                                                  out.data_ptr(), _ops()._stream()), "bsi_hip_quantize_trunc_to_int64")
    return out


def _ints_round(x2d: torch.Tensor, decimal_places: int) -> torch.Tensor:
    """round half away from zero of x * 10^dec (the decimal builders' rule, bsiFunctions.cpp:760-774)."""
    out = torch.empty(x2d.shape, dtype=torch.int64, device=x2d.device)
    if x2d.numel():
        check(lib.bsi_hip_quantize_round_to_int64(x2d.data_ptr(), _lib.DTYPE_F32, x2d.numel(), 10.0 ** int(decimal_places),
                                                  out.data_ptr(), _ops()._stream()), "bsi_hip_quantize_round_to_int64")
    return out


class _Sliced:
    """Bit-sliced rows: planes [rows, S, W], per-row slice weights, and what the stats functions report."""

    def __init__(self, ints: torch.Tensor, threshold: float):
        ops = _ops()
        self.rows, self.d = int(ints.shape[0]), int(ints.shape[1])
        self.words, self.weights, self.S, self.negative = ops._planes_from_ints(ints)
        self.W = int(self.words.shape[2])
        self.threshold = float(threshold)
        self._report = None

    def report(self) -> Tuple[int, int, int]:
        """(slices, verbatim slices, bytes): a slice is kept verbatim (W words) unless its density flag asks for the
        EWAH stream, whose length then counts."""
        if self._report is None:
            ops = _ops()
            flat = self.words.reshape(self.rows * self.S, self.W)
            if flat.shape[0] == 0:
                self._report = (0, 0, 0)
            else:
                _comp, _off, comp_len, flags = ops.ewah_compress_slices(flat, self.threshold)
                compressed = int((flags != 0).sum().item())
                total = int(flat.shape[0])
                self._report = (total, total - compressed, int(comp_len.to(torch.int64).sum().item()) * 8)
        return self._report

    def mem_bytes(self) -> int:
        return self.report()[2]


def _raw_dot(a: _Sliced, b: _Sliced) -> Tuple[torch.Tensor, int]:
    """Exact integer dot products of the rows of ``a`` with the rows of ``b`` as float64 [a.rows, b.rows], and the
    kernel's duration in ns (device events)."""
    ops = _ops()
    ops._check(a.d == b.d, f"vector lengths differ: {a.d} vs {b.d}")
    out = torch.zeros((a.rows, b.rows), dtype=torch.float64, device=a.words.device)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    if a.rows and b.rows and a.d:
        check(lib.bsi_hip_dot_weighted_f64(a.words.data_ptr(), a.weights.data_ptr(), a.S, a.W, b.words.data_ptr(),
                                           _lib.LAYOUT_CANONICAL, b.weights.data_ptr(), b.S, b.rows, a.rows, None,
                                           b.rows, out.data_ptr(), ops._stream()), "bsi_hip_dot_weighted_f64")
    e1.record()
    e1.synchronize()
    return out, int(e0.elapsed_time(e1) * 1.0e6)


def _scale(decimals: int) -> float:
    return 10.0 ** decimals if decimals > 0 else 1.0


# --------------------------------------------------------------------------- one pair of vectors


def dot_product(m: torch.Tensor, n: torch.Tensor, precision_factor: float):
    """bsiFunctions.cpp:249-340, :386-389: integers ``(long)(x * (long)precision_factor)``, exact dot, divided by
    ``float(precision_factor * precision_factor)``.  -> (result, dot ns, bytes of vector 1, bytes of vector 2)."""
    a, b = _vec(m, "m"), _vec(n, "n")
    factor = float(int(precision_factor))
    sa = _Sliced(_ints_trunc(a.unsqueeze(0), factor), 0.2)
    sb = _Sliced(_ints_trunc(b.unsqueeze(0), factor), 0.2)
    raw, ns = _raw_dot(sa, sb)
    pf = np.float32(precision_factor)
    return float(raw.item()) / float(np.float32(pf * pf)), ns, sa.mem_bytes(), sb.mem_bytes()


def dot_product_decimal(m: torch.Tensor, n: torch.Tensor, decimalPlaces: int):
    """bsiFunctions.cpp:342-384, :391-394: decimal builder on both vectors, exact dot / 10^(2 dec)."""
    a, b = _vec(m, "m"), _vec(n, "n")
    sa = _Sliced(_ints_round(a.unsqueeze(0), decimalPlaces), 0.2)
    sb = _Sliced(_ints_round(b.unsqueeze(0), decimalPlaces), 0.2)
    raw, ns = _raw_dot(sa, sb)
    return float(raw.item()) / _scale(2 * int(decimalPlaces)), ns, sa.mem_bytes(), sb.mem_bytes()


def random_number_dot_product_bsi(m: torch.Tensor, n: torch.Tensor):
    """bsiFunctions.cpp:121-155, :396-399: integers ``(long)x``, exact dot. -> (result, ns)."""
    a, b = _vec(m, "m"), _vec(n, "n")
    raw, ns = _raw_dot(_Sliced(_ints_trunc(a.unsqueeze(0), 1.0), 0.2), _Sliced(_ints_trunc(b.unsqueeze(0), 1.0), 0.2))
    return float(raw.item()), ns


def _timed_int_dot(ia: torch.Tensor, ib: torch.Tensor) -> Tuple[int, int]:
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    res = (ia * ib).sum()
    e1.record()
    e1.synchronize()
    return int(res.item()), int(e0.elapsed_time(e1) * 1.0e6)


def random_number_dot_product_vector(m: torch.Tensor, n: torch.Tensor):
    """bsiFunctions.cpp:95-119, :401-404: the plain-integer baseline of random_number_dot_product_bsi, a 64-bit sum
    of products of ``(long)x``. -> (result, ns)."""
    a, b = _vec(m, "m"), _vec(n, "n")
    _ops()._check(a.numel() <= b.numel(), "n is shorter than m")
    ia, ib = _ints_trunc(a.unsqueeze(0), 1.0)[0], _ints_trunc(b.unsqueeze(0), 1.0)[0]
    return _timed_int_dot(ia, ib[: ia.numel()])


def _capacity(n: int) -> int:
    """Capacity of a std::vector grown by n push_backs from empty (doubling): the byte counts vector_dot_product
    reports are capacity * 8 (bsiFunctions.cpp:186-192)."""
    cap = 0
    while cap < n:
        cap = max(1, cap * 2)
    return cap


def vector_dot_product(m: torch.Tensor, n: torch.Tensor, precision_factor: float):
    """bsiFunctions.cpp:157-208, :416-424: the plain-integer baseline of dot_product.  Integers
    ``(int64)(x * (int64)precision_factor)``; the reference accumulates in an ``int`` (``auto res = 0``), so the sum is
    reduced to 32 bits, and it is NOT divided by the factor.  -> (result, ns, bytes 1, bytes 2, 64, 64)."""
    a, b = _vec(m, "m"), _vec(n, "n")
    _ops()._check(a.numel() <= b.numel(), "n is shorter than m")
    factor = float(int(precision_factor))
    ia, ib = _ints_trunc(a.unsqueeze(0), factor)[0], _ints_trunc(b.unsqueeze(0), factor)[0]
    res, ns = _timed_int_dot(ia, ib[: ia.numel()])
    res = (res + (1 << 31)) % (1 << 32) - (1 << 31)
    return res, ns, _capacity(a.numel()) * 8, _capacity(b.numel()) * 8, 64, 64


def vector_dot_product_no_precison(m: torch.Tensor, n: torch.Tensor):
    """bsiFunctions.cpp:210-247, :406-414: ``(int16)x`` on both sides, 64-bit sum.
    -> (result, ns, bytes 1, bytes 2, 16, 16).  Values beyond int16 are undefined in the reference; here they wrap."""
    a, b = _vec(m, "m"), _vec(n, "n")
    _ops()._check(a.numel() <= b.numel(), "n is shorter than m")
    ia = _ints_trunc(a.unsqueeze(0), 1.0)[0].to(torch.int16).to(torch.int64)
    ib = _ints_trunc(b.unsqueeze(0), 1.0)[0].to(torch.int16).to(torch.int64)
    res, ns = _timed_int_dot(ia, ib[: ia.numel()])
    return res, ns, a.numel() * 2, b.numel() * 2, 16, 16


# --------------------------------------------------------------------------- one query against many keys


class PrebuiltBSIKeys(object):
    """bsiFunctions.cpp:480-486."""

    name = "PrebuiltBSIKeys"

    def __init__(self, sliced: _Sliced, decimal_places: int, threshold: float):
        self.sliced = sliced
        self.decimalPlaces = int(decimal_places)
        self.d = sliced.d
        self.num_keys = sliced.rows
        self.threshold = float(threshold)


class PrebuiltBSIQuery(object):
    """bsiFunctions.cpp:492-496."""

    name = "PrebuiltBSIQuery"

    def __init__(self, sliced: _Sliced, decimal_places: int, threshold: float):
        self.sliced = sliced
        self.decimalPlaces = int(decimal_places)
        self.threshold = float(threshold)


def _keys(cap) -> PrebuiltBSIKeys:
    _ops()._check(isinstance(cap, PrebuiltBSIKeys), "Invalid BSI keys capsule")
    return cap


def _query(cap) -> PrebuiltBSIQuery:
    _ops()._check(isinstance(cap, PrebuiltBSIQuery), "Invalid BSI query capsule")
    return cap


def batch_dot_product(q: torch.Tensor, K: torch.Tensor, decimalPlaces: int, threshold: float = 0.2):
    """bsiFunctions.cpp:426-478: decimal builder on the query and on every key row, out[r] = exact dot / 10^(2 dec)
    as float64.  -> (out [num_keys] float64 on the CPU, dot ns, bytes of the query, bytes of the first key)."""
    ops = _ops()
    ops._check(isinstance(q, torch.Tensor) and q.dim() == 1, "q must be 1D")
    ops._check(isinstance(K, torch.Tensor) and K.dim() == 2, "K must be 2D")
    ops._check(q.shape[0] == K.shape[1], "q.size(0) must equal K.size(1)")
    sq = _Sliced(_ints_round(_vec(q, "q").unsqueeze(0), decimalPlaces), threshold)
    sk = _Sliced(_ints_round(_mat(K, "K"), decimalPlaces), threshold)
    raw, ns = _raw_dot(sq, sk)
    first = _Sliced(_ints_round(_mat(K[:1], "K"), decimalPlaces), threshold).mem_bytes() if K.shape[0] else 0
    return raw[0].cpu() / _scale(2 * int(decimalPlaces)), ns, sq.mem_bytes(), first  # IEEE division, on the host


def build_bsi_keys(K: torch.Tensor, decimal_places: int, compress_threshold: float = 0.2):
    """bsiFunctions.cpp:567-610. -> (capsule, bytes, num_keys, d)."""
    _ops()._check(isinstance(K, torch.Tensor) and K.dim() == 2, "K must be 2D [num_keys, d]")
    sliced = _Sliced(_ints_round(_mat(K, "K"), decimal_places), compress_threshold)
    cap = PrebuiltBSIKeys(sliced, decimal_places, compress_threshold)
    return cap, sliced.mem_bytes(), cap.num_keys, cap.d


def build_bsi_query(q: torch.Tensor, decimal_places: int, compress_threshold: float = 0.2):
    """bsiFunctions.cpp:612-649. -> (capsule, bytes, slices)."""
    _ops()._check(isinstance(q, torch.Tensor) and q.dim() == 1, "q must be 1D [d]")
    sliced = _Sliced(_ints_round(_vec(q, "q").unsqueeze(0), decimal_places), compress_threshold)
    return PrebuiltBSIQuery(sliced, decimal_places, compress_threshold), sliced.mem_bytes(), sliced.S


def batch_dot_product_prebuilt(q: torch.Tensor, keyset_cap, query_threshold: float = -1.0):
    """bsiFunctions.cpp:651-701. -> (out float64 [num_keys] on the CPU, total ns, build ns, dot ns, query bytes)."""
    ops = _ops()
    ops._check(isinstance(q, torch.Tensor) and q.dim() == 1, "q must be 1D [d]")
    keys = _keys(keyset_cap)
    ops._check(q.shape[0] == keys.d, "q.size(0) must equal keys' dimension")
    thr = float(query_threshold) if query_threshold >= 0.0 else keys.threshold
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    sq = _Sliced(_ints_round(_vec(q, "q").unsqueeze(0), keys.decimalPlaces), thr)
    e1.record()
    e1.synchronize()
    build_ns = int(e0.elapsed_time(e1) * 1.0e6)
    raw, dot_ns = _raw_dot(sq, keys.sliced)
    out = raw[0].cpu() / _scale(2 * keys.decimalPlaces)
    return out, build_ns + dot_ns, build_ns, dot_ns, sq.mem_bytes()


def batch_dot_product_prebuilt_capsule(query_cap, keyset_cap):
    """bsiFunctions.cpp:703-731. -> (out float64 [num_keys] on the CPU, dot ns, 0, dot ns, query bytes)."""
    query, keys = _query(query_cap), _keys(keyset_cap)
    raw, dot_ns = _raw_dot(query.sliced, keys.sliced)
    out = raw[0].cpu() / _scale(query.decimalPlaces + keys.decimalPlaces)
    return out, dot_ns, 0, dot_ns, query.sliced.mem_bytes()


# --------------------------------------------------------------------------- statistics, files, debug


def _stats_dict(total: int, verbatim: int) -> dict:
    compressed = total - verbatim if total >= verbatim else 0
    return {"total_slices": total, "verbatim_slices": verbatim, "compressed_slices": compressed,
            "compressed_pct": (compressed * 100.0 / total) if total else 0.0,
            "verbatim_pct": (verbatim * 100.0 / total) if total else 0.0}


def keyset_slice_stats(keyset_cap) -> dict:
    """bsiFunctions.cpp:502-523."""
    keys = _keys(keyset_cap)
    total, verbatim, _ = keys.sliced.report()
    out = {"num_vectors": keys.num_keys}
    out.update(_stats_dict(total, verbatim))
    return out


def tensor_slice_stats(tensor: torch.Tensor, decimal_places: int, compress_threshold: float = 0.2,
                       signed_input: bool = True) -> dict:
    """bsiFunctions.cpp:525-565.  ``signed_input=False`` asks bsiCPP for its unsigned builder; the slices built here
    are those of the signed one either way (a non-negative vector has an all-zero sign slice)."""
    _ops()._check(isinstance(tensor, torch.Tensor) and tensor.dim() == 1, "tensor must be 1D [n]")
    sliced = _Sliced(_ints_round(_vec(tensor, "tensor").unsqueeze(0), decimal_places), compress_threshold)
    total, verbatim, nbytes = sliced.report()
    out = _stats_dict(total, verbatim)
    out.update({"memory_bytes": nbytes, "decimal_places": int(decimal_places),
                "compress_threshold": float(compress_threshold), "signed_input": bool(signed_input)})
    return out


def _as_device_keyset(keys: PrebuiltBSIKeys):
    ops = _ops()
    h = ops.PrebuiltBSIKeysCUDA()
    s = keys.sliced
    h.num_keys, h.d, h.W, h.Sb, h.fixed = s.rows, s.d, s.W, s.S, False
    h.decimals, h.threshold = keys.decimalPlaces, keys.threshold
    h.words, h.layout, h.slice_weights = s.words, _lib.LAYOUT_CANONICAL, s.weights
    return h


def keyset_size_on_disk(keyset_cap):
    """bsiFunctions.cpp:776-790. -> (bytes in memory, bytes save_keyset writes)."""
    keys = _keys(keyset_cap)
    return keys.sliced.mem_bytes(), _ops().keyset_size_on_disk_cuda(_as_device_keyset(keys))[1]


def save_keyset(keyset_cap, out_dir: str) -> None:
    """bsiFunctions.cpp:792-808 writes one bsiCPP ``.hb`` file per key and slice; that container is defined by the
    absent library, so this writes the build's own keyset file (``keyset.bsik``, see save_keyset_cuda), which
    load_keyset_cuda reads back."""
    _ops().save_keyset_cuda(_as_device_keyset(_keys(keyset_cap)), os.fspath(out_dir))


def debug_bsi_query_words(query_cap):
    """bsiFunctions.cpp:733-756. -> (words int64 [slices, W] on the CPU, rows, offset, decimals, twos_complement)."""
    query = _query(query_cap)
    s = query.sliced
    return s.words[0].cpu(), s.d, 0, query.decimalPlaces, bool(int(s.negative[0].item()) != 0)
