"""ctypes/numpy front end of the CPU oracle (``bsi_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the CPU-baseline
leg of the benchmark, never by the library.  Each function forwards to the C restatement of
the reference block named in its docstring (paths relative to the reference's
``bsi_ops/csrc/cuda/``); the decimal-mode functions and the scalar entry points at the end are
numpy.  Every function is pinned by an independent check in ``tests/test_oracle_*.py`` (none is
"parity unpinned"; of the scalar entry points only the VALUES are restated: their byte counts and
slice statistics come out of the bsiCPP containers, which the reference's tree does not hold).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libbsi_oracle.so")

_i64p = np.ctypeslib.ndpointer(np.int64, flags="C_CONTIGUOUS")
_u64p = np.ctypeslib.ndpointer(np.uint64, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    override = os.environ.get("BSI_ORACLE_LIBRARY")  # e.g. the sanitized build, `make -C oracle libbsi_oracle_ubsan.so`
    if override is None and not os.path.exists(_SO):
        build()
    L = ctypes.CDLL(override if override is not None else _SO)
    L.bsi_oracle_round_half_away.restype = ctypes.c_int64
    L.bsi_oracle_round_half_away.argtypes = [ctypes.c_double]
    L.bsi_oracle_round_to_int64.restype = None
    L.bsi_oracle_round_to_int64.argtypes = [_f32p, ctypes.c_int64, ctypes.c_int, _i64p]
    L.bsi_oracle_compute_shift.restype = ctypes.c_int
    L.bsi_oracle_compute_shift.argtypes = [ctypes.c_uint64, ctypes.c_double, ctypes.c_int, ctypes.c_int, ctypes.c_float]
    L.bsi_oracle_shift_clamp.restype = ctypes.c_int64
    L.bsi_oracle_shift_clamp.argtypes = [ctypes.c_int64, ctypes.c_int, ctypes.c_int]
    L.bsi_oracle_quantize_fixed.restype = None
    L.bsi_oracle_quantize_fixed.argtypes = [_f32p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                            ctypes.c_int, ctypes.c_float, _i64p, _i32p, _f32p]
    L.bsi_oracle_pack.restype = None
    L.bsi_oracle_pack.argtypes = [_i64p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int64, _u64p]
    L.bsi_oracle_slice_weights.restype = None
    L.bsi_oracle_slice_weights.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, _f32p]
    L.bsi_oracle_compress_flags.restype = None
    L.bsi_oracle_compress_flags.argtypes = [_u64p, ctypes.c_int, ctypes.c_int, ctypes.c_double, _i32p]
    L.bsi_oracle_ewah_size.restype = None
    L.bsi_oracle_ewah_size.argtypes = [_u64p, ctypes.c_int, ctypes.c_int, _i32p, _u64p]
    L.bsi_oracle_ewah_emit.restype = None
    L.bsi_oracle_ewah_emit.argtypes = [_u64p, ctypes.c_int, ctypes.c_int, _i32p, _u64p, _u64p, _i32p]
    L.bsi_oracle_ewah_decompress.restype = None
    L.bsi_oracle_ewah_decompress.argtypes = [_u64p, ctypes.c_int, ctypes.c_int, _u64p]
    L.bsi_oracle_dot_fixed.restype = None
    L.bsi_oracle_dot_fixed.argtypes = [_u64p, _f32p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _u64p, _f32p,
                                       ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_float, ctypes.c_int64,
                                       ctypes.c_void_p, ctypes.c_void_p]
    L.bsi_oracle_num_threads.restype = ctypes.c_int
    L.bsi_oracle_num_threads.argtypes = []
    _lib = L
    return L


def num_threads() -> int:
    return int(lib().bsi_oracle_num_threads())


def round_half_away(x: float) -> int:
    """bsi_cuda_kernels_quant.cuh:24-29."""
    return int(lib().bsi_oracle_round_half_away(float(x)))


def round_to_int64(x: np.ndarray, decimal_places: int) -> np.ndarray:
    """bsi_cuda_kernels_quant.cuh:110-121."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.int64)
    lib().bsi_oracle_round_to_int64(x.reshape(-1), x.size, int(decimal_places), out.reshape(-1))
    return out


def compute_shift(max_abs: int, sum_abs: float, count: int, fixed_bits: int, clip_k: float = 0.0) -> int:
    """bsi_cuda_kernels_quant.cuh:82-108."""
    return int(lib().bsi_oracle_compute_shift(int(max_abs), float(sum_abs), int(count), int(fixed_bits), float(clip_k)))


def shift_clamp(v: int, shift: int, fixed_bits: int) -> int:
    """bsi_cuda_kernels_quant.cuh:205-226."""
    return int(lib().bsi_oracle_shift_clamp(int(v), int(shift), int(fixed_bits)))


def quantize_fixed(x: np.ndarray, decimal_places: int, fixed_bits: int, chunk_scale: bool, clip_k: float = 0.0):
    """Fixed-bit quantiser, bsi_cuda_kernels_quant.cuh:255-488.

    Returns ``(ints[Q,d] int64, shifts int32, scales float32)``; shifts/scales are
    ``[Q, ceil(d/256)]`` with ``chunk_scale`` and ``[Q]`` without.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    Q, d = x.shape
    chunks = (d + 255) // 256 if chunk_scale else 1
    ints = np.zeros((Q, d), dtype=np.int64)
    shifts = np.zeros((Q, chunks), dtype=np.int32)
    scales = np.ones((Q, chunks), dtype=np.float32)
    if Q and d:
        lib().bsi_oracle_quantize_fixed(x.reshape(-1), Q, d, int(decimal_places), int(fixed_bits), int(bool(chunk_scale)),
                                        float(clip_k), ints.reshape(-1), shifts.reshape(-1), scales.reshape(-1))
    if not chunk_scale:
        shifts, scales = shifts[:, 0].copy(), scales[:, 0].copy()
    return ints, shifts, scales


def pack(ints: np.ndarray, slices: int) -> np.ndarray:
    """bsi_cuda_kernels_pack.cuh:129-174 -> words ``[Q, slices, W64]`` uint64."""
    ints = np.ascontiguousarray(ints, dtype=np.int64)
    Q, d = ints.shape
    W = (d + 63) // 64 if d > 0 else 1
    words = np.zeros((Q, slices, W), dtype=np.uint64)
    if Q and d:
        lib().bsi_oracle_pack(ints.reshape(-1), Q, d, int(slices), W, words.reshape(-1))
    return words


def slice_weights(S: int, offset: int = 0, twos: bool = True) -> np.ndarray:
    """bsi_cuda.cpp:217-236."""
    out = np.zeros(S, dtype=np.float32)
    lib().bsi_oracle_slice_weights(int(S), int(offset), int(bool(twos)), out)
    return out


def compress_flags(words: np.ndarray, threshold: float) -> np.ndarray:
    """bsi_cuda_kernels_ewah.cuh:47-69,84-102; ``words`` is ``[S, W]``."""
    words = np.ascontiguousarray(words, dtype=np.uint64)
    S, W = words.shape
    flags = np.zeros(S, dtype=np.int32)
    lib().bsi_oracle_compress_flags(words.reshape(-1), S, W, float(threshold), flags)
    return flags


def ewah_encode(words: np.ndarray, flags: np.ndarray):
    """bsi_cuda_kernels_ewah.cuh:118-232 -> ``(stream uint64[total], off int64[S], len int32[S])``."""
    words = np.ascontiguousarray(words, dtype=np.uint64)
    flags = np.ascontiguousarray(flags, dtype=np.int32)
    S, W = words.shape
    sizes = np.zeros(S, dtype=np.uint64)
    lib().bsi_oracle_ewah_size(words.reshape(-1), S, W, flags, sizes)
    off = np.zeros(S, dtype=np.uint64)
    off[1:] = np.cumsum(sizes)[:-1]
    total = int(sizes.sum())
    out = np.zeros(max(total, 1), dtype=np.uint64)
    lens = np.zeros(S, dtype=np.int32)
    lib().bsi_oracle_ewah_emit(words.reshape(-1), S, W, flags, off, out, lens)
    assert (lens.astype(np.uint64) == sizes).all(), "size pass and emit pass disagree"
    return out[:total], off.astype(np.int64), lens


def ewah_decompress(stream: np.ndarray, W: int) -> np.ndarray:
    """bsi_cuda_kernels_ewah.cuh:5-33."""
    stream = np.ascontiguousarray(stream, dtype=np.uint64)
    out = np.zeros(W, dtype=np.uint64)
    buf = stream if stream.size else np.zeros(1, dtype=np.uint64)
    lib().bsi_oracle_ewah_decompress(buf, int(stream.size), int(W), out)
    return out


def dot_fixed(A: np.ndarray, qscale: np.ndarray, B: np.ndarray, bscale: np.ndarray, scale_inv: float,
              want_ints: bool = True, want_out: bool = True):
    """bsi_cuda_kernels_dot.cuh:1384-1542.

    ``A`` ``[Q,Sa,W]`` uint64, ``qscale`` ``[Q,chunks]`` or ``[Q]`` (row scale, broadcast over chunks),
    ``B`` ``[R,Sb,W]``, ``bscale`` ``[R]``.  Returns ``(chunk_ints int32 [Q,R,chunks] | None, out f32 [Q,R] | None)``.
    """
    A = np.ascontiguousarray(A, dtype=np.uint64)
    B = np.ascontiguousarray(B, dtype=np.uint64)
    Q, Sa, W = A.shape
    R, Sb, Wb = B.shape
    assert W == Wb
    chunks = (W + 3) // 4
    qscale = np.asarray(qscale, dtype=np.float32)
    if qscale.ndim == 1:
        qscale = np.repeat(qscale[:, None], chunks, axis=1)
    qscale = np.ascontiguousarray(qscale)
    assert qscale.shape == (Q, chunks), (qscale.shape, (Q, chunks))
    bscale = np.ascontiguousarray(bscale, dtype=np.float32)
    assert bscale.shape == (R,)
    ints = np.zeros((Q, R, chunks), dtype=np.int32) if want_ints else None
    out = np.zeros((Q, R), dtype=np.float32) if want_out else None
    lib().bsi_oracle_dot_fixed(A.reshape(-1), qscale.reshape(-1), chunks, Sa, W, B.reshape(-1), bscale, Sb, R, Q,
                               ctypes.c_float(scale_inv), R,
                               ints.ctypes.data if ints is not None else None,
                               out.ctypes.data if out is not None else None)
    return ints, out


def scale_inv(dec_q: int, dec_k: int) -> np.float32:
    """bsi_cuda.cpp:709-711: ``(float)(1 / 10^(dec_q + dec_k))``."""
    total = int(dec_q) + int(dec_k)
    return np.float32(1.0 / (10.0 ** total)) if total > 0 else np.float32(1.0)


def build_queries(x: np.ndarray, decimal_places: int = 2, fixed_bits: int = 7, clip_k: float = 0.0):
    """Query side of bsi_vector_cuda.cpp:971-1064: chunk scales iff ``W64 % 4 == 0``.

    Returns dict(words, ints, shifts, scales, chunk_scale, slice_weights).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    d = x.shape[1]
    W = (d + 63) // 64 if d > 0 else 1
    chunk = (W % 4) == 0
    ints, shifts, scales = quantize_fixed(x, decimal_places, fixed_bits, chunk, clip_k)
    return dict(words=pack(ints, fixed_bits), ints=ints, shifts=shifts, scales=scales, chunk_scale=chunk,
                slice_weights=slice_weights(fixed_bits))


def build_keys(k: np.ndarray, decimal_places: int = 2, fixed_bits: int = 6, clip_k: float = 0.0):
    """Key side of bsi_vector_cuda.cpp:971-1197 (``for_keys``): per-row scale, ``Bw[r,j] = w_j * 2^shift_r``."""
    k = np.ascontiguousarray(k, dtype=np.float32)
    ints, shifts, scales = quantize_fixed(k, decimal_places, fixed_bits, False, clip_k)
    bw = slice_weights(fixed_bits)[None, :] * scales[:, None]
    return dict(words=pack(ints, fixed_bits), ints=ints, shifts=shifts, scales=scales, slice_weights=bw.astype(np.float32))


# --------------------------------------------------------------------------- decimal (data-dependent slice count) mode


def choose_total_slices(any_non_zero: bool, max_abs: int) -> int:
    """bsi_vector_cuda.cpp:746-754 with ``fixed_bits == 0``: magnitude bits of the largest |value| plus two,
    at most 64; two slices for an all-zero input."""
    if not any_non_zero:
        return 2
    return min(64, max(1, int(max_abs).bit_length()) + 2)


def build_decimal(x: np.ndarray, decimal_places: int = 2):
    """Batch builder without fixed bits, bsi_vector_cuda.cpp:565-577 (round half away of ``x * 10^dec``, no
    scale) and :1088-1166: one slice count for the whole batch from its largest magnitude, the low ``S`` bits
    of every two's-complement value packed into planes, and per row the two's-complement slice weights when
    the row holds a negative value, the unsigned ones otherwise.  The 1-D builder (:778-852) is the Q = 1 case.

    Returns dict(words [Q,S,W] uint64, ints [Q,d] int64, S, slice_weights [Q,S] float32, negative [Q] bool).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    Q, d = x.shape
    ints = round_to_int64(x, decimal_places) if x.size else np.zeros((Q, d), dtype=np.int64)
    any_non_zero = bool(Q > 0 and np.any(ints != 0))
    max_abs = int(np.abs(ints).max()) if any_non_zero else 0
    S = max(1, choose_total_slices(any_non_zero, max_abs))
    negative = (ints < 0).any(axis=1) if Q > 0 else np.zeros((0,), dtype=bool)
    w_twos, w_unsigned = slice_weights(S, 0, True), slice_weights(S, 0, False)
    weights = np.where(negative[:, None], w_twos[None, :], w_unsigned[None, :]).astype(np.float32)
    return dict(words=pack(ints, S), ints=ints, S=S, slice_weights=weights, negative=negative)


def dot_weighted(A: np.ndarray, Aw: np.ndarray, B: np.ndarray, Bw: np.ndarray, scale_inv: float) -> np.ndarray:
    """The weighted-slice dot every non-chunk-scale call computes, bsi_cuda_kernels_dot.cuh:150-187:
    ``out[q,r] = (sum over i, j, w of popcount(A[q,i,w] & B[r,j,w]) * (Aw[q,i] * Bw[r,j])) * scale_inv`` with the
    coefficient ``Aw * Bw`` a float32 product.  The reference adds the terms in fp32 in an order fixed by its
    launch shape (strided per thread, then shuffle trees); every term is an integer times a power of two, so
    this restatement adds them exactly (float64; exact while the sum of magnitudes stays below 2^53) and
    rounds once to float32 -- the value any fp32 order approximates to within its rounding error.
    """
    A = np.ascontiguousarray(A, dtype=np.uint64)
    B = np.ascontiguousarray(B, dtype=np.uint64)
    Aw = np.ascontiguousarray(Aw, dtype=np.float32)
    Bw = np.ascontiguousarray(Bw, dtype=np.float32)
    Q, Sa, W = A.shape
    R, Sb, Wb = B.shape
    assert W == Wb and Aw.shape == (Q, Sa) and Bw.shape == (R, Sb)
    out = np.zeros((Q, R), dtype=np.float32)
    for q in range(Q):
        # cnt[r, i, j] = sum_w popcount(A[q,i,w] & B[r,j,w])
        cnt = np.zeros((R, Sa, Sb), dtype=np.int64)
        for i in range(Sa):
            cnt[:, i, :] = np.bitwise_count(A[q, i][None, None, :] & B).sum(axis=2, dtype=np.int64)
        coeff = (Aw[q][None, :, None] * Bw[:, None, :]).astype(np.float32)          # float32 products
        acc = (cnt.astype(np.float64) * coeff.astype(np.float64)).sum(axis=(1, 2))   # exact
        out[q] = acc.astype(np.float32) * np.float32(scale_inv)
    return out


def int8_digits(ints: np.ndarray, S: int) -> np.ndarray:
    """Base-128 digits of S-bit two's-complement values, ``[ceil(S/7), ...]`` int64: the low digits are the
    unsigned 7-bit groups, the top digit the remaining bits with their sign, so that
    ``value = sum_j digit_j * 128^j`` and every digit fits an int8.  No counterpart in the reference: this is the
    operand form of the matrix-core route for decimal-mode operands."""
    v = np.asarray(ints, dtype=np.int64)
    n = (int(S) + 6) // 7
    out = np.zeros((n,) + v.shape, dtype=np.int64)
    for j in range(n - 1):
        out[j] = (v >> (7 * j)) & 127
    out[n - 1] = v >> (7 * (n - 1))  # arithmetic shift keeps the sign
    return out


# --------------------------------------------------------------------------- the scalar entry points (values only)


def trunc_scaled(x: np.ndarray, factor: float) -> np.ndarray:
    """``static_cast<long>(x * (long)factor)`` (bsi_ops/bsiFunctions.cpp:265-271, :165-170): the product is a
    float (float times long converts the long), the conversion goes towards zero."""
    return (np.asarray(x, dtype=np.float32) * np.float32(int(factor))).astype(np.int64)


def scalar_dot_product(m: np.ndarray, n: np.ndarray, precision_factor: float) -> float:
    """bsi_ops/bsiFunctions.cpp:249-340: exact dot of the truncated integers over
    ``float(precision_factor * precision_factor)`` (a float product), in double."""
    raw = int(trunc_scaled(m, precision_factor).astype(object) @ trunc_scaled(n, precision_factor).astype(object))
    pf = np.float32(precision_factor)
    return float(raw) / float(np.float32(pf * pf))


def scalar_dot_product_decimal(m: np.ndarray, n: np.ndarray, decimal_places: int) -> float:
    """bsi_ops/bsiFunctions.cpp:342-384: exact dot of the rounded integers (half away from zero, the builders'
    rule) over ``10^(2 dec)`` (1 when dec = 0), in double."""
    raw = int(round_to_int64(np.asarray(m, dtype=np.float32), decimal_places).astype(object)
              @ round_to_int64(np.asarray(n, dtype=np.float32), decimal_places).astype(object))
    total = 2 * int(decimal_places)
    return float(raw) / (10.0 ** total if total > 0 else 1.0)


def scalar_batch_dot_product(q: np.ndarray, K: np.ndarray, decimal_places: int) -> np.ndarray:
    """bsi_ops/bsiFunctions.cpp:426-478: scalar_dot_product_decimal of q with every row of K, float64 [num_keys]."""
    return np.array([scalar_dot_product_decimal(q, row, decimal_places) for row in np.asarray(K)], dtype=np.float64)


def scalar_vector_dot_product(m: np.ndarray, n: np.ndarray, precision_factor: float) -> int:
    """bsi_ops/bsiFunctions.cpp:157-208: the plain-integer baseline, accumulated in an ``int`` (``auto res = 0``),
    hence reduced to 32 bits, and not divided by the factor."""
    raw = int(trunc_scaled(m, precision_factor).astype(object) @ trunc_scaled(n, precision_factor).astype(object))
    return (raw + (1 << 31)) % (1 << 32) - (1 << 31)

