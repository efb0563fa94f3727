"""Python mirror of the reference ``bsi_ops`` extension module for the GPU tensor-dot path.

Same function names, argument meaning, return tuples and error behaviour as the pybind module the
reference registers in ``bsi_ops/csrc/cuda/bsi_cuda.cpp:1010-1078`` (and the module shell in
``bsi_ops/bsiFunctions.cpp:810-847``), so the reference's microbenchmarks and its
``BSIQuantizedLinear`` call it unchanged (``import bsipytorch_amd.bsi_ops as bsi_ops`` or the
top-level ``bsi_ops`` shim).  Handles are opaque objects with the reference's capsule names; they
own torch tensors, so device memory is released when the handle is garbage collected.

Every function forwards to ``libbsi_hip.so`` through its C ABI; torch is used for device memory
and the current stream only.  Fixed-bit mode (queries 7 bits with per-256-element chunk scales,
keys 6 bits with a per-row scale) is the default; the reference's environment names override it:
``BSI_FIXED_BITS``, ``BSI_FIXED_BITS_QUERIES``, ``BSI_FIXED_BITS_KEYS``, ``BSI_FIXED_CHUNK_SCALE``,
``BSI_FIXED_CLIP_K``, ``BSI_PROFILE``, ``BSI_DEBUG``, ``BSI_DOT_DEBUG``.  Flags that select NVIDIA
code paths (``BSI_TC_DOT``, ``BSI_TC_TMA``, ``BSI_TC_CPASYNC``, ``BSI_TC_R_SWEEP``,
``BSI_TC_FIXED_INT``, ``BSI_CUSTOM_QUANT``, ``BSI_FUSED_QPACK``, ``BSI_PACK_ONESHOT``, ``BSI_Q_TILE``,
``BSI_R_TILE``) are accepted and ignored.  Two flags are new: ``BSI_DOT_CORE`` = ``auto`` | ``mfma`` |
``valu`` and ``BSI_KEY_LAYOUT`` = ``tiled`` | ``canonical``.
"""
from __future__ import annotations

import ctypes
import json
import os
import sys
import threading
from typing import List, Optional

import torch

from . import _lib
from ._lib import check, lib

# --------------------------------------------------------------------------- flags


_ENV_DATA = getattr(os.environ, "_data", None)   # CPython on POSIX: the bytes-keyed dict behind os.environ
_ENV_KEYS: dict = {}


def fast_getenv(name: str, default: str) -> str:
    """os.environ.get for the per-call switches (read on every forward, as the reference reads its own): a plain dict
    lookup instead of os.environ's encode/decode round trip, which costs a forward of 100 layers half a millisecond."""
    if _ENV_DATA is None:
        return os.environ.get(name, default)
    key = _ENV_KEYS.get(name)
    if key is None:
        key = _ENV_KEYS[name] = os.fsencode(name)
    v = _ENV_DATA.get(key)
    return default if v is None else os.fsdecode(v)


def _env_int(name: str, default: Optional[int]) -> Optional[int]:
    s = os.environ.get(name)
    if s is None:
        return default
    try:
        return int(s)
    except ValueError:
        return 0  # atoi semantics


def _clamp_bits(v: int) -> int:
    # bsi_vector_cuda.cpp:254-276: <= 0 disables, otherwise clamp to [2, 63]
    if v <= 0:
        return 0
    return min(63, max(2, v))


_flag_cache: dict = {}


def _flags() -> dict:
    """Environment flags, read once per process like the reference's function-local statics."""
    if _flag_cache:
        return _flag_cache
    base = _env_int("BSI_FIXED_BITS", None)
    q = _env_int("BSI_FIXED_BITS_QUERIES", None)
    k = _env_int("BSI_FIXED_BITS_KEYS", None)
    # default (nothing set): fixed76 chunk-scale; an explicit 0 selects the decimal builder
    bits_q = _clamp_bits(q if q is not None else (base if base is not None else 7))
    bits_k = _clamp_bits(k if k is not None else (base if base is not None else 6))
    clip = 0.0
    try:
        clip = float(os.environ.get("BSI_FIXED_CLIP_K", "0") or 0)
    except ValueError:
        clip = 0.0
    core = os.environ.get("BSI_DOT_CORE", "auto").strip().lower()
    layout = os.environ.get("BSI_KEY_LAYOUT", "tiled").strip().lower()
    _flag_cache.update(
        bits_q=bits_q,
        bits_k=bits_k,
        chunk_scale=(_env_int("BSI_FIXED_CHUNK_SCALE", 1) or 0) != 0,
        clip_k=clip if clip > 0.0 else 0.0,
        profile=(_env_int("BSI_PROFILE", 0) or 0) != 0,
        debug=os.environ.get("BSI_DEBUG") is not None,
        dot_debug=(_env_int("BSI_DOT_DEBUG", 0) or 0) != 0,
        core={"auto": _lib.CORE_AUTO, "valu": _lib.CORE_VALU, "mfma": _lib.CORE_MFMA}.get(core, _lib.CORE_AUTO),
        tiled=(layout != "canonical"),
        key_image=(_env_int("BSI_KEY_INT8_IMAGE", 1) or 0) != 0,
        ewah_inline=(_env_int("BSI_EWAH_INLINE", 1) or 0) != 0,
        decimal_mfma=(_env_int("BSI_DECIMAL_MFMA", 1) or 0) != 0,
        image_tiled=(_env_int("BSI_KEY_IMAGE_TILED", 0) or 0) != 0,
        dot_split=(_env_int("BSI_DOT_SPLIT", 1) or 0) != 0,
    )
    return _flag_cache


def _reset_flag_cache() -> None:
    """Test hook: re-read the environment on the next call."""
    _flag_cache.clear()
    _DOT_DEBUG_PRINTED[0] = False


def _check(cond: bool, msg: str) -> None:
    # TORCH_CHECK surfaces as RuntimeError in Python
    if not cond:
        raise RuntimeError(msg)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_device_objects: dict = {}


def _stream() -> int:
    """Handle of torch's current stream on the current device (what every launch is enqueued on)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _device() -> torch.device:
    idx = torch.cuda.current_device() if _device_objects else -1
    dev = _device_objects.get(idx)
    if dev is None:
        _check(torch.cuda.is_available(), "bsi_ops: no GPU visible; the HIP path is the only path")
        idx = torch.cuda.current_device()
        dev = _device_objects[idx] = torch.device("cuda", idx)
    return dev


def _dtype_code(t: torch.Tensor) -> int:
    return {torch.float32: _lib.DTYPE_F32, torch.float16: _lib.DTYPE_F16, torch.bfloat16: _lib.DTYPE_BF16}[t.dtype]


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


# --------------------------------------------------------------------------- handles


class _Capsule:
    """Opaque handle; ``name`` is the reference's PyCapsule name."""

    name = ""

    def __repr__(self) -> str:  # pragma: no cover - cosmetic
        return f'<capsule object "{self.name}" at {hex(id(self))}>'


class PrebuiltBSIKeysCUDA(_Capsule):
    """bsi_cuda.cpp:153-177 (single Sb group, identity key order)."""

    name = "PrebuiltBSIKeysCUDA"

    def __init__(self):
        self.words: torch.Tensor = None          # canonical [R, Sb, W] or tiled [ceil(R/16), chunks, Sb, 64]
        self.layout = _lib.LAYOUT_CANONICAL
        self.ints8: Optional[torch.Tensor] = None  # cached int8 image of the same integers, or None: row-major
        self.ints8_tiled = False                   # [R, chunks*256], or tiled [ceil(R/64), 2 chunks, 64, 128] (flat)
        self.slice_weights: torch.Tensor = None  # [R, Sb] float32
        self.shifts: torch.Tensor = None         # [R] int32 (fixed-bit keys only)
        self.fixed = True                        # False: decimal-mode keys (slice count from the data, canonical planes)
        self.digits8: Optional[torch.Tensor] = None  # decimal keys: int8 digit images [ceil(Sb/7), R, chunks*256]
        self.Sb = 0
        self.W = 0
        self.d = 0
        self.num_keys = 0
        self.decimals = 0
        self.threshold = 0.2


class PrebuiltBSIQueryBatchCUDA(_Capsule):
    """bsi_cuda.cpp:202-211."""

    name = "PrebuiltBSIQueryBatchCUDA"

    def __init__(self):
        self.words: torch.Tensor = None          # [Q, Sa, W] int64
        self.slice_weights: torch.Tensor = None  # [Q, Sa] float32
        self.chunk_scales: Optional[torch.Tensor] = None  # [Q, chunks] float32 or None
        self.row_scales: Optional[torch.Tensor] = None    # [Q] float32 when there are no chunk scales
        self.ints8: Optional[torch.Tensor] = None         # [Q, chunks*256] int8 (MFMA operand) or None
        self.fixed = True                                 # False: decimal-mode batch (no scales; weighted-slice dot)
        self.digits8: Optional[torch.Tensor] = None       # decimal batch: int8 digit images [ceil(Sa/7), Q, chunks*256]
        self.Sa = 0
        self.W = 0
        self.decimals = 0
        self.Q = 0
        self.mem_bytes = 0


class PrebuiltBSIQueryBatchHybridCUDA(_Capsule):
    """A query batch whose slices are kept as EWAH streams only (the batched form of the hybrid query of
    bsi_cuda.cpp:386-431; the reference has no batched one): stream q * Sa + s is slice s of row q."""

    name = "PrebuiltBSIQueryBatchHybridCUDA"

    def __init__(self):
        self.comp_words: torch.Tensor = None     # int64 [total]: all streams, back to back
        self.comp_off: torch.Tensor = None       # int64 [Q * Sa]
        self.comp_len: torch.Tensor = None       # int32 [Q * Sa]
        self.flags: torch.Tensor = None          # int32 [Q * Sa]: 1 = the slice was run-length encoded
        self.slice_weights: torch.Tensor = None  # [Q, Sa] float32
        self.chunk_scales: Optional[torch.Tensor] = None
        self.row_scales: Optional[torch.Tensor] = None
        self.Sa = 0
        self.W = 0
        self.decimals = 0
        self.Q = 0
        self.mem_bytes = 0                       # bytes of the streams (+ offsets, lengths, scales)
        self.verbatim_bytes = 0                  # bytes the same planes take verbatim


class PrebuiltBSIQueryCUDA(_Capsule):
    """bsi_cuda.cpp:183-192: one query row (a view into its batch)."""

    name = "PrebuiltBSIQueryCUDA"

    def __init__(self):
        self.dev_words: torch.Tensor = None      # [S, W]
        self.slice_weights: torch.Tensor = None  # [S]
        self.chunk_scales: Optional[torch.Tensor] = None  # [chunks]
        self.row_scale: Optional[torch.Tensor] = None     # [] when no chunk scales
        self.ints8: Optional[torch.Tensor] = None         # [chunks*256]
        self.fixed = True                                 # False: decimal-mode row (no scale)
        self.digits8: Optional[torch.Tensor] = None       # decimal row: int8 digit images [ceil(S/7), chunks*256]
        self.S = 0
        self.W = 0
        self.rows = 0
        self.decimals = 0
        self.twos_complement = False
        self.mem_bytes = 0
        # hybrid builder only
        self.comp_words: Optional[torch.Tensor] = None
        self.comp_off: Optional[torch.Tensor] = None
        self.comp_len: Optional[torch.Tensor] = None


def tensor_build_key(t: torch.Tensor, *extra):
    """What identifies the query build of ``t``: its storage address, shape, dtype, version counter and the flags the
    build depends on -- or None when the contents cannot be tracked (a tensor made under ``torch.inference_mode()``
    keeps no version counter), in which case nothing is shared and every call builds anew."""
    if t.is_inference():
        return None
    f = _flags()
    return (t.data_ptr(), tuple(t.shape), t.dtype, t._version, f["bits_q"], f["chunk_scale"], f["clip_k"]) + extra


def capture_id() -> int:
    """Identifier of the graph capture the current stream is recording into, 0 when it is not capturing."""
    if not _capturing():
        return 0
    cid = ctypes.c_ulonglong(0)
    check(lib.bsi_hip_stream_capture_id(_stream(), ctypes.byref(cid)), "bsi_hip_stream_capture_id")
    return int(cid.value)


def _capsule(obj, cls, what: str):
    _check(isinstance(obj, cls), what)
    return obj


# --------------------------------------------------------------------------- builder

_last_build_profile = [0, 0, 0]


def get_last_query_build_profile_cuda():
    """(quantize_ns, pack_ns, total_ns) of the last query-batch build; zeros unless BSI_PROFILE=1
    (bsi_cuda.cpp:1036-1041).  The chunk-scale build is one fused kernel here, reported as pack_ns."""
    return tuple(_last_build_profile)


def reset_last_query_build_profile_cuda() -> None:
    _last_build_profile[:] = [0, 0, 0]


def cuda_builder_version() -> str:
    return "HIP_BUILDER_GFX950_FIXED76 " + _lib.version()


CUDA_BUILDER_VERSION = cuda_builder_version()


_slice_weight_cache: dict = {}


_gpu_present: Optional[bool] = None  # torch.cuda.is_available() costs 2 us a call and cannot change within a process


def _capturing() -> bool:
    global _gpu_present
    if _gpu_present is None:
        _gpu_present = bool(torch.cuda.is_available())
    return _gpu_present and torch.cuda.is_current_stream_capturing()


def _slice_weights(S: int, offset: int, twos: bool, device) -> torch.Tensor:
    # bsi_cuda.cpp:217-236; cached per device like make_slice_weights_cuda_cached (bsi_vector_cuda.cpp:48-88).
    # Callers must not modify the returned tensor.
    key = (int(S), int(offset), bool(twos), str(device))
    t = _slice_weight_cache.get(key)
    if t is None:
        if _capturing():
            # A host-to-device copy is not allowed while the stream records a graph, and a tensor made here only gets
            # its values when the graph runs: computed on the device (powers of two as integer shifts, exact) and
            # kept out of the cache, which eager callers read.
            e = torch.arange(int(S), device=device, dtype=torch.int64) + int(offset)
            t = torch.ones(int(S), device=device, dtype=torch.float32)
            for lo in (0, 62, 124):
                t = t * torch.bitwise_left_shift(torch.ones_like(e), (e - lo).clamp(0, 62)).to(torch.float32)
            t = torch.where(e < 0, torch.zeros_like(t), t)
            if twos and S > 0:
                t[S - 1] = -t[S - 1]
            return t
        w = [float(2.0 ** (offset + i)) if offset + i >= 0 else 0.0 for i in range(S)]
        if twos and S > 0:
            w[S - 1] = -w[S - 1]
        t = torch.tensor(w, dtype=torch.float32, device=device)
        _slice_weight_cache[key] = t
    return t


def _as_build_input(x: torch.Tensor, device) -> torch.Tensor:
    x = x.detach()
    if x.device != device:
        x = x.to(device)
    if x.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        x = x.to(torch.float32)
    return x.contiguous()


def _build_fixed(x2d: torch.Tensor, decimal_places: int, fixed_bits: int, chunk_scale: bool, want_ints8: bool):
    """One call of bsi_hip_build_fixed -> (words [Q,S,W] int64, shifts, scales, ints8 | None)."""
    f = _flags()
    dev = x2d.device
    Q, d = x2d.shape
    W = (d + 63) // 64 if d > 0 else 1
    chunks = (d + 255) // 256 if d > 0 else 0
    if Q > 0 and d > 0:   # the build kernels write every word, shift and scale: no fill passes
        alloc_i, alloc_f = torch.empty, torch.empty
    else:
        alloc_i, alloc_f = torch.zeros, torch.ones
    words = alloc_i((Q, fixed_bits, W), dtype=torch.int64, device=dev)
    if chunk_scale:
        shifts = alloc_i((Q, chunks), dtype=torch.int32, device=dev)
        scales = alloc_f((Q, chunks), dtype=torch.float32, device=dev)
    else:
        shifts = alloc_i((Q,), dtype=torch.int32, device=dev)
        scales = alloc_f((Q,), dtype=torch.float32, device=dev)
    ints8 = None
    if want_ints8 and fixed_bits <= 8 and Q > 0 and d > 0:
        ints8 = torch.empty((Q, ((W + 3) // 4) * 256), dtype=torch.int8, device=dev)
    if Q > 0 and d > 0:
        check(lib.bsi_hip_build_fixed(x2d.data_ptr(), _dtype_code(x2d), Q, d, int(decimal_places), fixed_bits,
                                      1 if chunk_scale else 0, f["clip_k"], words.data_ptr(), shifts.data_ptr(),
                                      scales.data_ptr(), _ptr(ints8), _stream()), "bsi_hip_build_fixed")
    return words, shifts, scales, ints8


def _build_decimal(x2d: torch.Tensor, decimal_places: int):
    """Decimal mode (``BSI_FIXED_BITS*=0``), bsi_vector_cuda.cpp:565-577 + :1088-1166: round ``x * 10^dec`` half
    away from zero, one slice count for the batch from its largest magnitude (:746-754), low ``S`` bits of the
    two's-complement values packed, and per row the two's-complement weights iff the row holds a negative value.
    -> (words [Q,S,W] int64, slice_weights [Q,S] float32, S, row_negative [Q] int32).
    Reads one scalar back from the device to size the planes, as the reference does (``.item()``, :1092-1096)."""
    dev = x2d.device
    Q, d = x2d.shape
    st = _stream()
    ints = torch.empty((Q, d), dtype=torch.int64, device=dev)
    if Q > 0 and d > 0:
        check(lib.bsi_hip_quantize_round_to_int64(x2d.data_ptr(), _dtype_code(x2d), Q * d, 10.0 ** int(decimal_places),
                                                  ints.data_ptr(), st), "bsi_hip_quantize_round_to_int64")
    return _planes_from_ints(ints)


def _planes_from_ints(ints: torch.Tensor):
    """Two's-complement planes of an int64 matrix [Q, d] with the decimal builder's slice rule
    (bsi_vector_cuda.cpp:746-754): -> (words [Q,S,W] int64, slice_weights [Q,S] float32, S, row_negative [Q])."""
    dev = ints.device
    Q, d = ints.shape
    W = (d + 63) // 64 if d > 0 else 1
    st = _stream()
    max_abs = torch.empty((1,), dtype=torch.int64, device=dev)
    negative = torch.zeros((Q,), dtype=torch.int32, device=dev)
    check(lib.bsi_hip_decimal_stats(ints.data_ptr() if Q > 0 and d > 0 else None, Q, d, max_abs.data_ptr(),
                                    negative.data_ptr() if Q > 0 else None, st), "bsi_hip_decimal_stats")
    m = int(max_abs.item()) & 0xFFFFFFFFFFFFFFFF  # |INT64_MIN| comes back as an unsigned 2^63
    S = 2 if m == 0 else min(64, m.bit_length() + 2)
    words = torch.zeros((Q, S, W), dtype=torch.int64, device=dev)
    if Q > 0 and d > 0:
        check(lib.bsi_hip_pack_bits_batch(ints.data_ptr(), Q, d, S, W, words.data_ptr(), st), "bsi_hip_pack_bits_batch")
    w_twos, w_unsigned = _slice_weights(S, 0, True, dev), _slice_weights(S, 0, False, dev)
    weights = torch.where(negative.bool().unsqueeze(1), w_twos.unsqueeze(0), w_unsigned.unsqueeze(0)).contiguous()
    return words, weights, S, negative


_MAX_DIGIT_PAIRS = 9  # above this the digit GEMM does more work than the popcount kernel saves


def _digit_images(words: torch.Tensor) -> Optional[torch.Tensor]:
    """int8 digit images [ceil(S/7), rows, chunks*256] of decimal-mode planes [rows, S, W] for the matrix cores
    (bsi_hip_planes_to_int8_digits), or None when the flag is off, the operand is empty or a row has more than
    2^17 elements (the int32 sums of the digit products could overflow)."""
    rows, S, W = words.shape
    if not _flags()["decimal_mfma"] or rows == 0 or W > 2048:
        return None
    out = torch.empty(((S + 6) // 7, rows, ((W + 3) // 4) * 256), dtype=torch.int8, device=words.device)
    check(lib.bsi_hip_planes_to_int8_digits(words.data_ptr(), rows, S, W, out.data_ptr(), _stream()),
          "bsi_hip_planes_to_int8_digits")
    return out


_expanded_cache: dict = {}
_warmed_query_caches: set = set()


def _expanded_slice_weights(base: torch.Tensor, Q: int, bits: int, dev) -> torch.Tensor:
    """[Q, bits] copies of the base slice weights; constant per (Q, bits, device), so built once
    (the reference caches its slice weights the same way, bsi_vector_cuda.cpp:48-88)."""
    key = (int(Q), int(bits), str(dev))
    t = _expanded_cache.get(key)
    if t is None:
        if len(_expanded_cache) > 64:
            _expanded_cache.clear()
            _warmed_query_caches.clear()
        t = base.unsqueeze(0).expand(Q, -1).contiguous()
        if _capturing():
            return t  # filled when the graph runs: not for the cache
        _expanded_cache[key] = t
    return t


def warm_query_build_caches(Q: int) -> None:
    """Creates the constant tensors a fixed-bit query build of Q rows reads (slice weights and their per-row copies),
    so that a build recorded into a HIP graph later finds them.  A forward that skips the builder when run eagerly
    (the fused few-rows kernel) calls this for the graph capture that does not skip it."""
    f = _flags()
    if f["bits_q"] == 0:
        return
    done = (int(Q), f["bits_q"], torch.cuda.current_device())
    if done in _warmed_query_caches or _capturing():
        return
    dev = _device()
    _expanded_slice_weights(_slice_weights(f["bits_q"], 0, True, dev), int(Q), f["bits_q"], dev)
    _warmed_query_caches.add(done)


def _build_query_batch(q2d: torch.Tensor, decimal_places: int) -> PrebuiltBSIQueryBatchCUDA:
    """bsi_vector_cuda.cpp:971-1064 (queries): chunk scales iff the flag is on and W64 % 4 == 0."""
    f = _flags()
    dev = _device()
    x = _as_build_input(q2d, dev)
    Q, d = x.shape
    W = (d + 63) // 64 if d > 0 else 1
    chunk_scale = f["chunk_scale"] and (W % 4 == 0)
    prof = f["profile"]
    if prof:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
    if f["bits_q"] == 0:  # decimal mode: the slice count follows the data; no scales
        words, weights, S, _neg = _build_decimal(x, decimal_places)
        if prof:
            e1.record()
            e1.synchronize()
            ns = int(e0.elapsed_time(e1) * 1.0e6)
            _last_build_profile[:] = [0, ns, ns]
        else:
            _last_build_profile[:] = [0, 0, 0]
        h = PrebuiltBSIQueryBatchCUDA()
        h.words, h.slice_weights, h.fixed = words, weights, False
        h.digits8 = _digit_images(words) if S <= 7 * _MAX_DIGIT_PAIRS else None
        h.Sa, h.W, h.decimals, h.Q = S, W, int(decimal_places), Q
        h.mem_bytes = words.numel() * 8 + weights.numel() * 4
        if f["debug"]:
            print(f"[BSI_HIP] build_bsi_queries_cuda_batch_data: Q={Q} slices={S} words_per_slice={W}")
        return h
    words, _shifts, scales, ints8 = _build_fixed(x, decimal_places, f["bits_q"], chunk_scale, want_ints8=True)
    if prof:
        e1.record()
        e1.synchronize()
        ns = int(e0.elapsed_time(e1) * 1.0e6)
        _last_build_profile[:] = [0, ns, ns]
    else:
        _last_build_profile[:] = [0, 0, 0]
    h = PrebuiltBSIQueryBatchCUDA()
    base = _slice_weights(f["bits_q"], 0, True, dev)
    h.words = words
    if chunk_scale:
        h.slice_weights = _expanded_slice_weights(base, Q, f["bits_q"], dev)
        h.chunk_scales = scales
    else:
        h.slice_weights = (base.unsqueeze(0) * scales.unsqueeze(1)).contiguous()
        h.row_scales = scales
    h.ints8 = ints8
    h.Sa = f["bits_q"]
    h.W = W
    h.decimals = int(decimal_places)
    h.Q = Q
    h.mem_bytes = words.numel() * 8 + h.slice_weights.numel() * 4
    if h.chunk_scales is not None and h.chunk_scales.numel() > 0:
        h.mem_bytes += h.chunk_scales.numel() * 4
    if f["debug"]:
        print(f"[BSI_HIP] build_bsi_queries_cuda_batch_data (fused): Q={Q} slices={h.Sa} words_per_slice={W}")
    return h


def build_bsi_queries_cuda_batch_packed(q2d: torch.Tensor, decimal_places: int, compress_threshold: float = 0.2):
    """bsi_cuda.cpp:346-379.  ``compress_threshold`` is accepted and unused, as in the reference."""
    _check(q2d.dim() == 2, "q must be 2D [Q, d]")
    return _build_query_batch(q2d, int(decimal_places))


def build_bsi_queries_cuda_batch(q2d: torch.Tensor, decimal_places: int, compress_threshold: float = 0.2) -> List:
    """bsi_cuda.cpp:272-344: one handle per row, all views into one batch build."""
    _check(q2d.dim() == 2, "q must be 2D [Q, d]")
    b = _build_query_batch(q2d, int(decimal_places))
    out = []
    for qi in range(b.Q):
        h = PrebuiltBSIQueryCUDA()
        h.S, h.W = b.Sa, b.W
        h.dev_words = b.words[qi]
        h.slice_weights = b.slice_weights[qi]
        h.fixed = b.fixed
        h.digits8 = b.digits8[:, qi] if b.digits8 is not None else None
        if b.chunk_scales is not None and b.chunk_scales.numel() > 0:
            h.chunk_scales = b.chunk_scales[qi]
        elif b.row_scales is not None:
            h.row_scale = b.row_scales[qi]
        h.ints8 = b.ints8[qi] if b.ints8 is not None else None
        h.mem_bytes = h.dev_words.numel() * 8
        h.rows = int(q2d.shape[1])
        h.decimals = int(decimal_places)
        h.twos_complement = False  # as the reference leaves it (bsi_cuda.cpp:303)
        out.append(h)
    return out


def _build_query_1d(q: torch.Tensor, decimal_places: int) -> PrebuiltBSIQueryCUDA:
    """bsi_vector_cuda.cpp:778-852 with fixed bits: one scale for the whole vector."""
    f = _flags()
    dev = _device()
    x = _as_build_input(q, dev).view(1, -1)
    if f["bits_q"] == 0:  # decimal mode: no scale; two's complement iff a negative value is present (:843)
        words, weights, S, neg = _build_decimal(x, decimal_places)
        h = PrebuiltBSIQueryCUDA()
        h.S, h.W, h.dev_words, h.rows, h.decimals, h.fixed = S, words.shape[2], words[0], x.shape[1], int(decimal_places), False
        h.twos_complement = bool(neg[0].item()) if x.shape[1] > 0 else False
        d8 = _digit_images(words) if S <= 7 * _MAX_DIGIT_PAIRS else None
        h.digits8 = d8[:, 0] if d8 is not None else None
        h.slice_weights = weights[0]
        h.mem_bytes = h.dev_words.numel() * 8
        return h
    words, _shifts, scales, ints8 = _build_fixed(x, decimal_places, f["bits_q"], False, want_ints8=True)
    h = PrebuiltBSIQueryCUDA()
    h.S = f["bits_q"]
    h.W = words.shape[2]
    h.dev_words = words[0]
    h.rows = x.shape[1]
    h.decimals = int(decimal_places)
    # two's complement only when a negative value is present (bsi_vector_cuda.cpp:843); the top
    # plane is empty otherwise, so the sign of its weight never matters
    h.twos_complement = bool((h.dev_words[h.S - 1] != 0).any().item()) if x.shape[1] > 0 else False
    h.slice_weights = _slice_weights(h.S, 0, h.twos_complement, dev) * scales[0]
    h.row_scale = scales[0]
    h.ints8 = ints8[0] if ints8 is not None else None
    h.mem_bytes = h.dev_words.numel() * 8
    return h


def build_bsi_query_cuda(q: torch.Tensor, decimal_places: int, compress_threshold: float = 0.2):
    """bsi_cuda.cpp:238-270 -> (handle, mem_bytes, S, W)."""
    _check(q.dim() == 1, "q must be 1D [d]")
    h = _build_query_1d(q, int(decimal_places))
    return h, int(h.mem_bytes), h.S, h.W


def ewah_compress_slices(words2d: torch.Tensor, compress_threshold: float):
    """Density flags + size pass + exclusive scan + emit pass for ``[S, W]`` words
    (bsi_vector_cuda.cpp:896-951).  Returns (comp_words, comp_off int64 [S], comp_len int32 [S], flags)."""
    S, W = words2d.shape
    dev = words2d.device
    st = _stream()
    counts = torch.empty((S,), dtype=torch.int64, device=dev)
    flags = torch.empty((S,), dtype=torch.int32, device=dev)
    sizes = torch.empty((S,), dtype=torch.int64, device=dev)
    check(lib.bsi_hip_slice_popcount_sum(words2d.data_ptr(), S, W, counts.data_ptr(), st), "bsi_hip_slice_popcount_sum")
    check(lib.bsi_hip_compress_flags_from_density(counts.data_ptr(), S, W, float(compress_threshold),
                                                  flags.data_ptr(), st), "bsi_hip_compress_flags_from_density")
    check(lib.bsi_hip_ewah_size(words2d.data_ptr(), S, W, flags.data_ptr(), sizes.data_ptr(), st), "bsi_hip_ewah_size")
    inclusive = sizes.cumsum(0)
    total = int(inclusive[-1].item()) if S > 0 else 0
    comp_off = (inclusive - sizes).contiguous()
    comp_words = torch.empty((max(total, 1),), dtype=torch.int64, device=dev)
    comp_len = torch.empty((S,), dtype=torch.int32, device=dev)
    check(lib.bsi_hip_ewah_emit(words2d.data_ptr(), S, W, flags.data_ptr(), comp_off.data_ptr(),
                                comp_words.data_ptr(), comp_len.data_ptr(), st), "bsi_hip_ewah_emit")
    return comp_words[:total], comp_off, comp_len, flags


def build_bsi_query_cuda_hybrid(q: torch.Tensor, decimal_places: int, compress_threshold: float = 0.2):
    """bsi_cuda.cpp:386-431: build, EWAH-compress every slice, then decode the streams back into the
    verbatim words the dot consumes.  mem_bytes counts both the stream and the words."""
    _check(q.dim() == 1, "q must be 1D [d]")
    h = _build_query_1d(q, int(decimal_places))
    planes = h.dev_words.contiguous()
    comp_words, comp_off, comp_len, _flags_dev = ewah_compress_slices(planes, float(compress_threshold))
    decoded = torch.zeros_like(planes)
    if comp_words.numel() > 0:
        check(lib.bsi_hip_ewah_decompress_batch(comp_words.data_ptr(), comp_off.data_ptr(), comp_len.data_ptr(),
                                                h.S, h.W, decoded.data_ptr(), _stream()),
              "bsi_hip_ewah_decompress_batch")
    else:
        decoded.copy_(planes)
    h.dev_words = decoded
    h.comp_words, h.comp_off, h.comp_len = comp_words, comp_off, comp_len
    h.mem_bytes = comp_words.numel() * 8 + decoded.numel() * 8
    return h, int(h.mem_bytes), h.S, h.W


def build_bsi_queries_cuda_batch_hybrid(q2d: torch.Tensor, decimal_places: int, compress_threshold: float = 0.2):
    """The batched hybrid query form: the fixed-bit build of build_bsi_queries_cuda_batch_packed, then every slice of
    every row EWAH-encoded at ``compress_threshold`` (density flag, size pass, scan, emit pass, as
    bsi_vector_cuda.cpp:896-951 does for the one query of build_bsi_query_cuda_hybrid) -- and only the streams are
    kept: the dot decodes them in its load stage.  Not in the reference, whose only hybrid form is one query that it
    decodes again right after encoding it (bsi_cuda.cpp:386-431)."""
    _check(q2d.dim() == 2, "q must be 2D [Q, d]")
    f = _flags()
    _check(2 <= f["bits_q"] <= 8, "the hybrid query batch needs fixed-bit queries of 2 to 8 bits")
    b = _build_query_batch(q2d, int(decimal_places))
    Q, Sa, W = b.words.shape
    _check(Q > 0, "Empty query batch")
    comp_words, comp_off, comp_len, flags = ewah_compress_slices(b.words.view(Q * Sa, W), float(compress_threshold))
    h = PrebuiltBSIQueryBatchHybridCUDA()
    h.comp_words, h.comp_off, h.comp_len, h.flags = comp_words, comp_off, comp_len, flags
    h.slice_weights, h.chunk_scales, h.row_scales = b.slice_weights, b.chunk_scales, b.row_scales
    h.Sa, h.W, h.decimals, h.Q = int(Sa), int(W), b.decimals, int(Q)
    scale_bytes = (b.chunk_scales.numel() if b.chunk_scales is not None else b.row_scales.numel()) * 4
    h.mem_bytes = comp_words.numel() * 8 + comp_off.numel() * 8 + comp_len.numel() * 4 + scale_bytes
    h.verbatim_bytes = b.words.numel() * 8 + scale_bytes
    return h


def _dot_ewah_batch(qb: "PrebuiltBSIQueryBatchHybridCUDA", keys: "PrebuiltBSIKeysCUDA", bias=None, chunk_ints=None):
    """bsi_hip_dot_ewah_batch on a hybrid query batch -> (out [Q, R] float32, ns)."""
    f = _flags()
    Q, R, Sa, W = qb.Q, keys.num_keys, qb.Sa, qb.W
    _check(2 <= keys.Sb <= 8 and keys.fixed, "the hybrid query batch needs fixed-bit keys of 2 to 8 bits")
    if qb.chunk_scales is not None and qb.chunk_scales.numel() > 0:
        _check(keys.W % 4 == 0 and qb.chunk_scales.shape[1] == keys.W // 4, "Chunk scale stride mismatch")
        scales, stride = qb.chunk_scales, int(qb.chunk_scales.shape[1])
    else:
        scales, stride = qb.row_scales, 1
    dev = qb.comp_words.device
    out = torch.empty((Q, R), dtype=torch.float32, device=dev)
    kptr, klayout = key_operand(keys, Q, Sa, _lib.CORE_MFMA)
    ws_bytes = int(lib.bsi_hip_dot_ewah_batch_workspace_bytes(Q, W))
    ws = _get_workspace(ws_bytes, dev)
    if Q >= _SPLIT_MIN_Q and chunk_ints is None:
        _attach_split_scratch_for(dev, Q, R, W)
    prof = f["profile"]
    if prof:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
    check(lib.bsi_hip_dot_ewah_batch(qb.comp_words.data_ptr(), qb.comp_off.data_ptr(), qb.comp_len.data_ptr(), Sa, W,
                                     scales.data_ptr(), stride, kptr, klayout, keys.slice_weights.data_ptr(), keys.Sb, R, Q,
                                     _scale_inv(qb.decimals, keys.decimals), R, _ptr(bias), out.data_ptr(), _ptr(chunk_ints),
                                     _ptr(ws), ws_bytes, _stream()), "bsi_hip_dot_ewah_batch")
    ns = 0
    if prof:
        e1.record()
        e1.synchronize()
        ns = int(e0.elapsed_time(e1) * 1.0e6)
    return out, ns


def _install_fixed_key_planes(h: "PrebuiltBSIKeysCUDA", words: torch.Tensor) -> None:
    """Derive the representations the dot reads from canonical fixed-bit planes [R, Sb, W]: the cached int8
    image (BSI_KEY_INT8_IMAGE) and the tiled planes (BSI_KEY_LAYOUT), or the canonical planes themselves."""
    f = _flags()
    dev = words.device
    R = h.num_keys
    if f["key_image"] and R > 0 and 2 <= h.Sb <= 8:
        # compute-bound shapes contract this image on the matrix cores; the planes stay the stored form
        if f["image_tiled"]:
            # tiled by 64 rows and half-chunks: a workgroup's key rows of a half-chunk are contiguous (off by
            # default: measured no faster than the row-major image, cache-resident or not)
            h.ints8 = torch.empty((int(lib.bsi_hip_int8_tiled_bytes(R, h.W)),), dtype=torch.int8, device=dev)
            h.ints8_tiled = True
            check(lib.bsi_hip_planes_to_int8_tiled(words.data_ptr(), R, h.Sb, h.W, h.ints8.data_ptr(), _stream()),
                  "bsi_hip_planes_to_int8_tiled")
        else:
            h.ints8 = torch.empty((R, ((h.W + 3) // 4) * 256), dtype=torch.int8, device=dev)
            h.ints8_tiled = False
            check(lib.bsi_hip_planes_to_int8(words.data_ptr(), R, h.Sb, h.W, h.ints8.data_ptr(), _stream()),
                  "bsi_hip_planes_to_int8")
    if f["tiled"] and R > 0:
        chunks = (h.W + 3) // 4
        tiled = torch.empty(((R + 15) // 16, chunks, h.Sb, 64), dtype=torch.int64, device=dev)
        check(lib.bsi_hip_tile_key_planes(words.data_ptr(), R, h.Sb, h.W, tiled.data_ptr(), _stream()),
              "bsi_hip_tile_key_planes")
        h.words, h.layout = tiled, _lib.LAYOUT_TILED16
    else:
        h.words, h.layout = words, _lib.LAYOUT_CANONICAL


def canonical_key_planes(keys: "PrebuiltBSIKeysCUDA") -> torch.Tensor:
    """The keyset's planes as canonical words [R, Sb, W] int64 on the device (undoes the 16-row tiling:
    word (r, j, 4c + g) sits at tile r // 16, chunk c, slice j, position g * 16 + r % 16)."""
    if keys.layout == _lib.LAYOUT_CANONICAL:
        return keys.words
    R, Sb, W = keys.num_keys, keys.Sb, keys.W
    tiles, chunks = keys.words.shape[0], keys.words.shape[1]
    t = keys.words.view(tiles, chunks, Sb, 4, 16).permute(0, 4, 2, 1, 3)  # [tile, r % 16, j, c, g]
    return t.reshape(tiles * 16, Sb, chunks * 4)[:R, :, :W].contiguous()


def build_bsi_keys_cuda(K: torch.Tensor, decimal_places: int, compress_threshold: float = 0.2):
    """bsi_cuda.cpp:863-910 (fixed-bit branch): per-row scale, Sb slices, ``Bw[r, j] = w_j * 2^shift_r``.
    Returns (handle, total_bytes_of_words, num_keys, d, W)."""
    _check(K.dim() == 2, "K must be 2D [num_keys, d]")
    f = _flags()
    dev = _device()
    x = _as_build_input(K, dev)
    R, d = x.shape
    if f["bits_k"] == 0:
        # Decimal mode.  The reference builds these keys row by row on the host with the bsiCPP library
        # (bsi_cuda.cpp:912-1000), which is not part of its tree; here the device builder the reference
        # uses for decimal queries is applied to the key matrix (one slice count for all rows, so one group
        # in identity order).  The integers each row stands for are the same rounded values either way.
        words, weights, S, _neg = _build_decimal(x, int(decimal_places))
        h = PrebuiltBSIKeysCUDA()
        h.num_keys, h.d, h.W, h.Sb, h.fixed = int(R), int(d), words.shape[2], S, False
        h.decimals, h.threshold = int(decimal_places), float(compress_threshold)
        h.words, h.layout, h.slice_weights = words, _lib.LAYOUT_CANONICAL, weights
        h.digits8 = _digit_images(words) if S <= 7 * _MAX_DIGIT_PAIRS else None
        if f["debug"]:
            print(f"[BSI_HIP] build_bsi_keys_cuda (decimal): R={R} slices={S} words_per_slice={h.W}")
        return h, int(words.numel() * 8), int(R), int(d), int(h.W)
    words, shifts, scales, _ = _build_fixed(x, int(decimal_places), f["bits_k"], False, want_ints8=False)
    h = PrebuiltBSIKeysCUDA()
    h.num_keys, h.d = int(R), int(d)
    h.W = words.shape[2]
    h.Sb = f["bits_k"]
    h.decimals = int(decimal_places)
    h.threshold = float(compress_threshold)
    h.shifts = shifts
    h.slice_weights = (_slice_weights(h.Sb, 0, True, dev).unsqueeze(0) * scales.unsqueeze(1)).contiguous()
    total_bytes = words.numel() * 8
    _install_fixed_key_planes(h, words)
    if f["debug"]:
        print(f"[BSI_HIP] build_bsi_keys_cuda: R={R} slices={h.Sb} words_per_slice={h.W} layout={h.layout}")
    return h, int(total_bytes), int(R), int(d), int(h.W)


def concat_keysets(keysets: List["PrebuiltBSIKeysCUDA"]) -> "PrebuiltBSIKeysCUDA":
    """One fixed-bit keyset holding the rows of several (same width, slice count and decimals), in order: the
    planes, slice weights and shifts are concatenated on the device and the dot's representations derived anew,
    so every row keeps exactly the bits it had.  No counterpart in the reference."""
    _check(len(keysets) > 0, "no keysets to concatenate")
    k0 = keysets[0]
    for k in keysets:
        _capsule(k, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule")
        _check(k.fixed and k.shifts is not None, "only fixed-bit keysets can be concatenated")
        _check((k.W, k.d, k.Sb, k.decimals) == (k0.W, k0.d, k0.Sb, k0.decimals), "keysets differ in shape or precision")
    h = PrebuiltBSIKeysCUDA()
    h.num_keys, h.d, h.W, h.Sb = sum(k.num_keys for k in keysets), k0.d, k0.W, k0.Sb
    h.decimals, h.threshold = k0.decimals, k0.threshold
    h.slice_weights = torch.cat([k.slice_weights for k in keysets]).contiguous()
    h.shifts = torch.cat([k.shifts for k in keysets]).contiguous()
    _install_fixed_key_planes(h, torch.cat([canonical_key_planes(k) for k in keysets]).contiguous())
    return h


def keyset_rows(keys: "PrebuiltBSIKeysCUDA", start: int, stop: int) -> "PrebuiltBSIKeysCUDA":
    """Rows start .. stop of a fixed-bit keyset as a keyset of their own that shares its memory (views); both
    bounds must be multiples of 64 or the end of the keyset, so that tiles are not split."""
    _capsule(keys, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule")
    _check(keys.fixed, "only fixed-bit keysets can be viewed by rows")
    _check(0 <= start < stop <= keys.num_keys and start % 64 == 0 and (stop % 64 == 0 or stop == keys.num_keys),
           "row bounds must be multiples of 64 within the keyset")
    h = PrebuiltBSIKeysCUDA()
    h.num_keys, h.d, h.W, h.Sb = stop - start, keys.d, keys.W, keys.Sb
    h.decimals, h.threshold, h.layout = keys.decimals, keys.threshold, keys.layout
    h.slice_weights, h.shifts = keys.slice_weights[start:stop], keys.shifts[start:stop]
    h.words = keys.words[start // 16:(stop + 15) // 16] if keys.layout == _lib.LAYOUT_TILED16 else keys.words[start:stop]
    if keys.ints8 is not None:
        h.ints8_tiled = keys.ints8_tiled
        if keys.ints8_tiled:
            tile = ((keys.W + 3) // 4) * 2 * 8192
            h.ints8 = keys.ints8[(start // 64) * tile:((stop + 63) // 64) * tile]
        else:
            h.ints8 = keys.ints8[start:stop]
    return h


# --------------------------------------------------------------------------- keyset files

_KEYSET_MAGIC = b"BSIKEYS1"
_KEYSET_FILE = "keyset.bsik"


def _keyset_header(keys: "PrebuiltBSIKeysCUDA") -> dict:
    return {"format": 1, "num_keys": keys.num_keys, "d": keys.d, "W": keys.W, "Sb": keys.Sb, "decimals": keys.decimals,
            "threshold": keys.threshold, "fixed": bool(keys.fixed), "byte_order": "little",
            "arrays": ["planes uint64 [num_keys, Sb, W]", "slice_weights float32 [num_keys, Sb]"]
                      + (["shifts int32 [num_keys]"] if keys.fixed else [])}


def keyset_size_on_disk_cuda(keyset_cuda_cap):
    """(bytes of the planes in device memory, bytes save_keyset_cuda would write); counterpart of
    keyset_size_on_disk (bsiFunctions.cpp:775-790) for device keysets."""
    keys = _capsule(keyset_cuda_cap, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule")
    plane_bytes = keys.num_keys * keys.Sb * keys.W * 8
    head = len(json.dumps(_keyset_header(keys)).encode())
    head = 16 + (head + 63) // 64 * 64
    return plane_bytes, head + plane_bytes + keys.num_keys * keys.Sb * 4 + (keys.num_keys * 4 if keys.fixed else 0)


def save_keyset_cuda(keyset_cuda_cap, out_dir: str) -> int:
    """Write a device keyset to ``out_dir/keyset.bsik`` and return the bytes written.  Counterpart of save_keyset
    (bsiFunctions.cpp:792-808), which writes one bsiCPP ``.hb`` file per key and slice; here one file holds an
    8-byte magic, the length of a JSON header, the header (padded to 64 bytes), then the packed planes
    (canonical [R, Sb, W] uint64, 0.75 byte per weight at 6 bits), the slice weights and the row shifts.
    The int8 image and the tiled planes are derived again on load."""
    keys = _capsule(keyset_cuda_cap, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule")
    os.makedirs(out_dir, exist_ok=True)
    head = json.dumps(_keyset_header(keys)).encode()
    head += b" " * ((-len(head)) % 64)
    planes = canonical_key_planes(keys).cpu().numpy()
    path = os.path.join(out_dir, _KEYSET_FILE)
    with open(path, "wb") as fh:
        fh.write(_KEYSET_MAGIC)
        fh.write(len(head).to_bytes(8, "little"))
        fh.write(head)
        fh.write(planes.astype("<i8", copy=False).tobytes())
        fh.write(keys.slice_weights.cpu().numpy().astype("<f4", copy=False).tobytes())
        if keys.fixed:
            fh.write(keys.shifts.cpu().numpy().astype("<i4", copy=False).tobytes())
    return os.path.getsize(path)


def load_keyset_cuda(out_dir: str):
    """Read ``out_dir/keyset.bsik`` back into a device keyset without re-quantising; returns the tuple
    build_bsi_keys_cuda returns: (handle, total_bytes_of_words, num_keys, d, W)."""
    import numpy as np

    path = os.path.join(out_dir, _KEYSET_FILE)
    with open(path, "rb") as fh:
        _check(fh.read(8) == _KEYSET_MAGIC, f"{path}: not a BSI keyset file")
        head_len = int.from_bytes(fh.read(8), "little")
        _check(0 < head_len <= (1 << 20), f"{path}: bad header length")
        meta = json.loads(fh.read(head_len).decode())
        _check(meta.get("format") == 1, f"{path}: unknown keyset format {meta.get('format')}")
        R, d, W, Sb = int(meta["num_keys"]), int(meta["d"]), int(meta["W"]), int(meta["Sb"])
        _check(R >= 0 and 1 <= Sb <= 64 and W == ((d + 63) // 64 if d > 0 else 1), f"{path}: inconsistent header")
        planes = np.fromfile(fh, dtype="<i8", count=R * Sb * W)
        weights = np.fromfile(fh, dtype="<f4", count=R * Sb)
        shifts = np.fromfile(fh, dtype="<i4", count=R) if meta["fixed"] else None
        _check(planes.size == R * Sb * W and weights.size == R * Sb and (shifts is None or shifts.size == R),
               f"{path}: truncated file")
    dev = _device()
    h = PrebuiltBSIKeysCUDA()
    h.num_keys, h.d, h.W, h.Sb = R, d, W, Sb
    h.decimals, h.threshold, h.fixed = int(meta["decimals"]), float(meta["threshold"]), bool(meta["fixed"])
    words = torch.from_numpy(planes.reshape(R, Sb, W)).to(dev)
    h.slice_weights = torch.from_numpy(weights.reshape(R, Sb)).to(dev)
    if h.fixed:
        h.shifts = torch.from_numpy(shifts).to(dev)
        _install_fixed_key_planes(h, words)
    else:
        h.words, h.layout = words, _lib.LAYOUT_CANONICAL
        h.digits8 = _digit_images(words) if Sb <= 7 * _MAX_DIGIT_PAIRS else None
    return h, int(R * Sb * W * 8), R, d, W


# --------------------------------------------------------------------------- dot

_DOT_DEBUG_PRINTED = [False]
_workspace: dict = {}
_FEW_ROWS_MAX_Q = 32  # up to here the dot streams the packed planes (bandwidth-bound); above, the int8 image


_retired_workspaces: list = []  # buffers whose address a recorded graph holds: never freed, never reused


def _get_workspace(nbytes: int, dev) -> Optional[torch.Tensor]:
    """Scratch memory for one dot on ``dev`` (derived int8 queries, digit products).  A launch recorded into a HIP
    graph has the buffer's address baked in, so a buffer that a capture has used is never given back to the
    allocator: when a later call needs more, a new one is added and the old one is kept alive for the replays."""
    if nbytes <= 0:
        return None
    rec = _workspace.get(dev)
    capturing = _capturing()
    if rec is None or rec["buf"].numel() < nbytes:
        _check(not capturing, "bsi_ops: this dot needs a larger workspace than exists; run it once before capturing a graph")
        if rec is not None and rec["captured"]:
            _retired_workspaces.append(rec["buf"])
        rec = _workspace[dev] = {"buf": torch.empty((nbytes,), dtype=torch.uint8, device=dev), "captured": False}
    if capturing:
        rec["captured"] = True
    return rec["buf"]


# D-split scratch of the int8-image dot (bsi_hip_dot_attach_split_scratch): device index -> {"capture": buffer,
# "eager": {stream: buffer}}.  One region per stream for eager launches (launches that share a region must not overlap
# on the GPU) and one for launches recorded into a graph; regions are never freed, since a recorded launch holds its
# region's address.  The library keeps the attachment per calling thread; _split_tls mirrors it to skip repeats.
_split_scratch: dict = {}
_split_tls = threading.local()
_SPLIT_MIN_Q = 33  # fewer query rows go to the few-rows kernels, which never split


def _new_split_region(dev) -> torch.Tensor:
    # zero-filled: the region's counters must start at zero, and every launch leaves them so
    return torch.zeros((int(lib.bsi_hip_dot_split_scratch_bytes()),), dtype=torch.uint8, device=dev)


def attach_split_scratch(dev=None) -> bool:
    """Attach this thread's D-split scratch region for the current stream of ``dev`` (default: the current device)
    before a dot is launched; returns whether one is attached.  BSI_DOT_SPLIT=0 never attaches one.  While a graph is
    being captured only a region that already exists is attached (a capture cannot allocate): the first eager call on
    a device creates the capture region too."""
    if not _flags()["dot_split"]:
        if getattr(_split_tls, "ptr", 0):
            check(lib.bsi_hip_dot_attach_split_scratch(None, 0), "bsi_hip_dot_attach_split_scratch")
            _split_tls.ptr = 0
        return False
    dev = _device() if dev is None else dev
    rec = _split_scratch.get(dev.index)
    capturing = _capturing()
    if rec is None:
        if capturing:
            buf = None
        else:
            rec = _split_scratch[dev.index] = {"capture": _new_split_region(dev), "eager": {}}
    if rec is not None:
        if capturing:
            buf = rec["capture"]
        else:
            st = _stream()
            buf = rec["eager"].get(st)
            if buf is None:
                buf = rec["eager"][st] = _new_split_region(dev)
    ptr = 0 if buf is None else buf.data_ptr()
    if getattr(_split_tls, "ptr", 0) != ptr or getattr(_split_tls, "dev", -1) != dev.index:
        check(lib.bsi_hip_dot_attach_split_scratch(ptr or None, 0 if buf is None else buf.numel()),
              "bsi_hip_dot_attach_split_scratch")
        _split_tls.ptr, _split_tls.dev = ptr, dev.index
    return buf is not None


_split_shapes: dict = {}  # (device index, Q, R, W) -> whether the launcher splits a dot of that shape


def _attach_split_scratch_for(dev, Q: int, R: int, W: int) -> None:
    """attach_split_scratch for the shapes the launcher would split, nothing for the others (a model's layers of a
    few hundred rows against thousands of keys never split: asking once per shape keeps the stream and capture
    look-ups out of every other forward).  The library's choice depends on the shape and the region's size only."""
    key = (dev.index, Q, R, W)
    use = _split_shapes.get(key)
    if use is None:
        if not attach_split_scratch(dev):
            return  # no region yet (a capture before any eager call): ask again next time
        tile, segments = ctypes.c_int(0), ctypes.c_int(0)
        check(lib.bsi_hip_dot_split_plan(R, Q, W, ctypes.byref(tile), ctypes.byref(segments)), "bsi_hip_dot_split_plan")
        _split_shapes[key] = segments.value > 1
    elif use:
        attach_split_scratch(dev)


def _scale_inv(dec_q: int, dec_k: int) -> float:
    # bsi_cuda.cpp:709-711: (float)(1.0 / 10^(dq + dk)); the C ABI takes it as float
    total = dec_q + dec_k
    return (1.0 / (10.0 ** total)) if total > 0 else 1.0


def key_operand(keys: "PrebuiltBSIKeysCUDA", Q: int, Sa: int, core: int):
    """(device pointer, layout code) of the key representation the dot should read for Q query rows:
    the packed planes while the call is bound by streaming them, the cached int8 image above."""
    if keys.ints8 is not None and core != _lib.CORE_VALU and Q > _FEW_ROWS_MAX_Q and 2 <= Sa <= 8:
        return keys.ints8.data_ptr(), (_lib.LAYOUT_INT8_TILED if keys.ints8_tiled else _lib.LAYOUT_INT8)
    return keys.words.data_ptr(), keys.layout


def _warm_region(next_keys, Q: int, Sa: int, core: int):
    """(pointer, bytes) of what a dot of Q query rows would read of ``next_keys``, or (None, 0)."""
    if next_keys is None or not next_keys.fixed:
        return None, 0
    if next_keys.ints8 is not None and core != _lib.CORE_VALU and Q > _FEW_ROWS_MAX_Q and 2 <= Sa <= 8:
        return next_keys.ints8.data_ptr(), next_keys.ints8.numel()
    return next_keys.words.data_ptr(), next_keys.words.numel() * 8


def _dot(words, ints8, scales, scale_stride, Sa, W, keys: PrebuiltBSIKeysCUDA, Q, decimals_q, chunk_ints=None, core=None,
         bias=None, warm_keys=None):
    f = _flags()
    dev = words.device
    R = keys.num_keys
    out = torch.empty((Q, R), dtype=torch.float32, device=dev)
    core = f["core"] if core is None else core
    # the reference's A/B switch between its tensor-core and popcount kernels is read on every call
    # (bsi_cuda_kernels_dot.cuh:2642); 0 selects the popcount core here
    if fast_getenv("BSI_TC_DOT", "1").strip() == "0" and words is not None:
        core = _lib.CORE_VALU
    ws = None
    ws_bytes = 0
    if ints8 is None:
        ws_bytes = int(lib.bsi_hip_dot_workspace_bytes(Q, W, core)) if (2 <= Sa <= 8 and 2 <= keys.Sb <= 8) else 0
        ws = _get_workspace(ws_bytes, dev)
    prof = f["profile"]
    if prof:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
    kptr, klayout = key_operand(keys, Q, Sa, core)
    if Q >= _SPLIT_MIN_Q and chunk_ints is None:
        _attach_split_scratch_for(dev, Q, R, W)
    if warm_keys is not None and chunk_ints is None:
        # the kernel also touches what the next layer's dot will read, so that it is cache-resident by then
        wptr, wbytes = _warm_region(warm_keys, Q, Sa, core)
        check(lib.bsi_hip_dot_bias_warm(words.data_ptr(), _ptr(ints8), scales.data_ptr(), scale_stride, Sa, W,
                                        kptr, klayout, keys.slice_weights.data_ptr(), keys.Sb, R, Q,
                                        _scale_inv(decimals_q, keys.decimals), R, _ptr(bias), out.data_ptr(), core,
                                        _ptr(ws), ws_bytes, wptr, wbytes, _stream()), "bsi_hip_dot_bias_warm")
    elif bias is not None and chunk_ints is None:
        check(lib.bsi_hip_dot_bias(words.data_ptr(), _ptr(ints8), scales.data_ptr(), scale_stride, Sa, W,
                                   kptr, klayout, keys.slice_weights.data_ptr(), keys.Sb, R, Q,
                                   _scale_inv(decimals_q, keys.decimals), R, bias.data_ptr(), out.data_ptr(), core,
                                   _ptr(ws), ws_bytes, _stream()), "bsi_hip_dot_bias")
    else:
        check(lib.bsi_hip_dot(words.data_ptr(), _ptr(ints8), scales.data_ptr(), scale_stride, Sa, W,
                              kptr, klayout, keys.slice_weights.data_ptr(), keys.Sb, R, Q,
                              _scale_inv(decimals_q, keys.decimals), R, out.data_ptr(), _ptr(chunk_ints), core,
                              _ptr(ws), ws_bytes, _stream()), "bsi_hip_dot")
        if bias is not None:
            check(lib.bsi_hip_add_bias(out.data_ptr(), bias.data_ptr(), Q, R, R, _stream()), "bsi_hip_add_bias")
    ns = 0
    if prof:
        e1.record()
        e1.synchronize()
        ns = int(e0.elapsed_time(e1) * 1.0e6)
    if f["dot_debug"] and not _DOT_DEBUG_PRINTED[0]:
        _DOT_DEBUG_PRINTED[0] = True
        print(f"[BSI_DOT] core={core} Sa={Sa} Sb={keys.Sb} Q={Q} R={R} W64={W} chunks={(W + 3) // 4} "
              f"layout={klayout} ints8={'yes' if ints8 is not None else 'no'}", file=sys.stderr)
    return out, ns


def _dot_weighted(words, slice_weights, Sa, W, keys: PrebuiltBSIKeysCUDA, Q, decimals_q, bias=None, q_digits=None,
                  q_image=None):
    """The weighted-slice dot: any operand pair that is not fixed-bit on both sides.  With int8 digit images on
    both sides (``q_digits`` [nq, Q, chunks*256] or the int8 image ``q_image`` of fixed-bit queries, pre-shifted by
    8 - Sa; the keys' own digits, or the int8 image of fixed-bit keys) it
    runs as one int8 GEMM on the matrix cores (bsi_hip_dot_digits), else on the popcount kernel
    (bsi_hip_dot_weighted); both give the exact sum rounded once, so the results are bit-identical."""
    f = _flags()
    R = keys.num_keys
    out = torch.empty((Q, R), dtype=torch.float32, device=words.device)
    Aw = slice_weights if slice_weights.is_contiguous() else slice_weights.contiguous()
    k_digits, nk, preshift, k_tiled = None, 0, 0, 0
    if q_digits is None and q_image is not None and 2 <= Sa <= 8:
        q_digits, preshift = q_image.unsqueeze(0), 8 - int(Sa)
    if keys.fixed and keys.ints8 is not None:
        k_digits, nk, preshift, k_tiled = keys.ints8, 1, preshift + 8 - keys.Sb, int(keys.ints8_tiled)
    elif not keys.fixed and keys.digits8 is not None:
        k_digits, nk = keys.digits8, int(keys.digits8.shape[0])
    use_digits = (f["decimal_mfma"] and f["core"] != _lib.CORE_VALU and q_digits is not None and k_digits is not None
                  and int(q_digits.shape[0]) * nk <= _MAX_DIGIT_PAIRS and W <= 2048)
    prof = f["profile"]
    if prof:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
    if use_digits:
        nq = int(q_digits.shape[0])
        qd = q_digits if q_digits.is_contiguous() else q_digits.contiguous()
        ws_bytes = int(lib.bsi_hip_dot_digits_workspace_bytes(Q, nq, R, nk))
        ws = _get_workspace(ws_bytes, words.device)
        check(lib.bsi_hip_dot_digits(qd.data_ptr(), nq, Aw.data_ptr(), int(Sa), k_digits.data_ptr(), nk, preshift,
                                     keys.slice_weights.data_ptr(), keys.Sb, int(W), R, Q, None,
                                     _scale_inv(decimals_q, keys.decimals), R, _ptr(bias), out.data_ptr(),
                                     ws.data_ptr(), ws_bytes, k_tiled, _stream()), "bsi_hip_dot_digits")
    else:
        check(lib.bsi_hip_dot_weighted(words.data_ptr(), Aw.data_ptr(), int(Sa), int(W), keys.words.data_ptr(),
                                       keys.layout, keys.slice_weights.data_ptr(), keys.Sb, R, Q, None,
                                       _scale_inv(decimals_q, keys.decimals), R, out.data_ptr(), _stream()),
              "bsi_hip_dot_weighted")
        if bias is not None:
            check(lib.bsi_hip_add_bias(out.data_ptr(), bias.data_ptr(), Q, R, R, _stream()), "bsi_hip_add_bias")
    ns = 0
    if prof:
        e1.record()
        e1.synchronize()
        ns = int(e0.elapsed_time(e1) * 1.0e6)
    if f["dot_debug"] and not _DOT_DEBUG_PRINTED[0]:
        _DOT_DEBUG_PRINTED[0] = True
        print(f"[BSI_DOT] core={'digits-mfma' if use_digits else 'weighted-valu'} Sa={Sa} Sb={keys.Sb} Q={Q} R={R} "
              f"W64={W} layout={keys.layout}", file=sys.stderr)
    return out, ns


FUSED_LINEAR_MAX_ROWS = 4
FUSED_LINEAR_QUERY_LDS_BYTES = 96 * 1024  # the kernel keeps the rows' int8 image and chunk scales in LDS


def _check_bias(bias, R: int, device) -> None:
    """A bias handed to a kernel is read through its device pointer: anything but a contiguous float32 tensor of [R] on
    the launch device is refused here (a host pointer would fault the GPU)."""
    if bias is not None:
        _check(isinstance(bias, torch.Tensor) and bias.is_cuda and bias.device == device and bias.dtype == torch.float32
               and bias.dim() == 1 and bias.numel() == R and bias.is_contiguous(),
               "bias must be a contiguous float32 CUDA tensor of [R] on the device of the call")


def device_bias(bias, device):
    """``bias`` if a kernel on ``device`` can add it in its epilogue (see _check_bias), else None: the caller then adds
    it afterwards."""
    if (bias is not None and bias.is_cuda and bias.device == device and bias.dtype == torch.float32 and bias.dim() == 1
            and bias.is_contiguous()):
        return bias
    return None


def can_fuse_linear_few_rows(x2d: torch.Tensor, keys: "PrebuiltBSIKeysCUDA") -> bool:
    """Whether linear_few_rows_cuda serves this call: a few rows, 7-or-so-bit chunk-scaled queries without
    clipping, fixed 6-plane tiled keys, the matrix-core route not switched off."""
    f = _flags()
    d = int(x2d.shape[1])
    return (0 < x2d.shape[0] <= FUSED_LINEAR_MAX_ROWS and x2d.is_cuda and x2d.is_contiguous()
            and x2d.dtype in (torch.float32, torch.float16, torch.bfloat16)
            and keys.fixed and keys.Sb == 6 and keys.layout == _lib.LAYOUT_TILED16 and keys.d == d
            and 2 <= f["bits_q"] <= 8 and f["chunk_scale"] and f["clip_k"] == 0.0 and ((d + 63) // 64) % 4 == 0
            and ((d + 255) // 256) * int(x2d.shape[0]) * 260 <= FUSED_LINEAR_QUERY_LDS_BYTES and f["core"] != _lib.CORE_VALU and not f["profile"]
            and fast_getenv("BSI_TC_DOT", "1").strip() != "0" and fast_getenv("BSI_FUSED_LINEAR", "1").strip() != "0")


def linear_few_rows_is_free(x2d: torch.Tensor, keys: "PrebuiltBSIKeysCUDA") -> bool:
    """Whether the fused kernel's query build hides entirely behind its key traffic for this shape
    (bsi_hip_linear_few_rows_upfront): then the one launch costs the GPU what the dot alone costs."""
    return bool(lib.bsi_hip_linear_few_rows_upfront(int(x2d.shape[0]), int(x2d.shape[1]), int(keys.num_keys)))


def linear_few_rows_cuda(x2d: torch.Tensor, keyset_cuda_cap, decimal_places: int, bias=None, _checked: bool = False) -> torch.Tensor:
    """out[Q, R] float32 = BSI dot of the rows of ``x2d`` (Q <= 4) with the keyset, query build included, in one
    launch (bsi_hip_linear_few_rows): what build_bsi_queries_cuda_batch_packed followed by
    batch_dot_product_multiquery_cuda_batch_caps returns, bit for bit.  Not in the reference."""
    keys = _capsule(keyset_cuda_cap, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule")
    if not _checked:  # the layer has asked can_fuse_linear_few_rows already
        _check(x2d.dim() == 2 and can_fuse_linear_few_rows(x2d, keys), "linear_few_rows_cuda: call not served by the fused kernel")
    _check(int(decimal_places) == keys.decimals,
           f"Decimal mismatch between queries and keys: q={int(decimal_places)} k={keys.decimals}")
    Q, R = int(x2d.shape[0]), keys.num_keys
    _check_bias(bias, R, x2d.device)
    out = torch.empty((Q, R), dtype=torch.float32, device=x2d.device)
    check(lib.bsi_hip_linear_few_rows(x2d.data_ptr(), _dtype_code(x2d), Q, int(x2d.shape[1]), int(decimal_places),
                                      _flags()["bits_q"], keys.words.data_ptr(), keys.slice_weights.data_ptr(), keys.Sb,
                                      R, _scale_inv(int(decimal_places), keys.decimals), R, _ptr(bias), out.data_ptr(),
                                      _stream()), "bsi_hip_linear_few_rows")
    return out


_last_linear_rebuilt = [False]  # whether the last linear_cuda call ran the query build (layer counters read it)
# device index -> {"bytes", "capture_buf", "captured", "capture": [key, input], "eager": {stream: (buffer, [key, input])}}
_linear_ws: dict = {}


def can_linear_one_call(x2d: torch.Tensor, keys: "PrebuiltBSIKeysCUDA") -> bool:
    """Whether linear_cuda serves this call: chunk-scaled fixed-bit queries without clipping against fixed-bit keys,
    the matrix-core route, no per-call profiling."""
    f = _flags()
    d = int(x2d.shape[1])
    return (x2d.shape[0] > 0 and x2d.is_cuda and x2d.is_contiguous()
            and x2d.dtype in (torch.float32, torch.float16, torch.bfloat16)
            and keys.fixed and keys.d == d and 2 <= f["bits_q"] <= 8 and f["chunk_scale"] and f["clip_k"] == 0.0
            and ((d + 63) // 64) % 4 == 0 and f["core"] != _lib.CORE_VALU and not f["profile"]
            and fast_getenv("BSI_TC_DOT", "1").strip() != "0" and fast_getenv("BSI_LINEAR_ONE_CALL", "1").strip() != "0")


def _linear_workspace(device, need: int, capturing: bool) -> dict:
    """linear_cuda's workspace record of ``device``: one buffer per stream for eager calls (forwards that run on
    different streams at the same time must not build into each other's operands) and one for launches recorded
    into a graph, (re)allocated outside captures when they are missing or smaller than ``need`` bytes.  A recorded
    launch holds the capture buffer's address, so once a capture has used it, it is kept alive for good: a larger
    need adds a new buffer for later captures and retires the old one instead of freeing it.  (Graphs replayed at the
    same time on different streams still share that one buffer: replay them on one stream.)"""
    ws = _linear_ws.get(device.index)
    if ws is None or ws["bytes"] < need:
        _check(not capturing, "linear_cuda: the workspace must exist before a graph is captured (run the forward once)")
        size = (max(need, 1 << 20) + 255) // 256 * 256
        if ws is not None and ws["captured"]:
            _retired_workspaces.append(ws["capture_buf"])
        ws = _linear_ws[device.index] = {"bytes": size, "captured": False,
                                         "capture_buf": torch.empty((size,), dtype=torch.uint8, device=device),
                                         "capture": [None, None], "eager": {}}
    if capturing:
        ws["captured"] = True
    return ws


_reserved_linear_shapes: set = set()
_linear_ws_need: dict = {}


def reserve_linear_workspace(x2d: torch.Tensor) -> None:
    """Make sure linear_cuda's workspace can take inputs of this shape.  A forward that runs eagerly on the few-rows
    kernel never calls linear_cuda, yet the same forward recorded into a graph may (build + dot is the faster pair
    there for longer rows), and a capture cannot allocate: the eager few-rows path calls this instead."""
    bits = _flags()["bits_q"]
    key = (x2d.device.index, int(x2d.shape[0]), int(x2d.shape[1]), bits)
    if key in _reserved_linear_shapes or not (2 <= bits <= 8) or _capturing():
        return
    _linear_workspace(x2d.device, int(lib.bsi_hip_linear_workspace_bytes(key[1], key[2], bits)), False)
    _reserved_linear_shapes.add(key)


def linear_cuda(x2d: torch.Tensor, keyset_cuda_cap, decimal_places: int, bias=None, warm_keys=None,
                _checked: bool = False) -> torch.Tensor:
    """out[Q, R] float32 of a BSI-linear layer in one library call (bsi_hip_linear): the query build into a workspace
    kept per device, then the dot, bit for bit what build_bsi_queries_cuda_batch_packed followed by
    batch_dot_product_multiquery_cuda_batch_caps returns.  A call on the very tensor the workspace was last built
    from (same storage, shape, dtype and version: the next layer fed the same activations) skips the build.
    Launches recorded into a HIP graph use a workspace of their own, so that replays and eager calls never find
    each other's builds.  Not in the reference; it takes the operand handles and half of the binding work out of
    an eager forward."""
    keys = _capsule(keyset_cuda_cap, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule")
    if not _checked:  # the layer has asked can_linear_one_call already
        _check(x2d.dim() == 2 and can_linear_one_call(x2d, keys), "linear_cuda: call not served by the one-call path")
    _check(int(decimal_places) == keys.decimals,
           f"Decimal mismatch between queries and keys: q={int(decimal_places)} k={keys.decimals}")
    f = _flags()
    Q, d, R = int(x2d.shape[0]), int(x2d.shape[1]), keys.num_keys
    _check_bias(bias, R, x2d.device)
    bits = f["bits_q"]
    need = _linear_ws_need.get((Q, d, bits))
    if need is None:  # a pure function of the shape: asked once per shape, not once per forward
        need = _linear_ws_need[(Q, d, bits)] = int(lib.bsi_hip_linear_workspace_bytes(Q, d, bits))
    capturing = _capturing()
    ws = _linear_workspace(x2d.device, need, capturing)
    st = _stream()
    if capturing:
        buf, slot = ws["capture_buf"], ws["capture"]
    else:
        mine = ws["eager"].get(st)
        if mine is None:  # first eager call on this stream (allocated under it, so freed in its order too)
            mine = ws["eager"][st] = (torch.empty((ws["bytes"],), dtype=torch.uint8, device=x2d.device), [None, None])
        buf, slot = mine
    key = tensor_build_key(x2d, int(decimal_places))
    if capturing and key is not None:
        # a build recorded by one capture is not part of another capture's graph: the capture's identifier is part
        # of what a recorded launch may reuse (a second capture starting on the same static input builds anew)
        key = key + (capture_id(),)
    rebuild = 0 if (key is not None and slot[0] == key) else 1
    slot[0], slot[1] = key, x2d  # holds the input, so that its address is not reused while the build stands for it
    wsptr = buf.data_ptr()
    out = torch.empty((Q, R), dtype=torch.float32, device=x2d.device)
    core = f["core"]
    kptr, klayout = key_operand(keys, Q, bits, core)
    if Q >= _SPLIT_MIN_Q:
        _attach_split_scratch_for(x2d.device, Q, R, (d + 63) // 64)
    wptr, wbytes = _warm_region(_capsule(warm_keys, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule") if warm_keys is not None
                                else None, Q, bits, core)
    check(lib.bsi_hip_linear(x2d.data_ptr(), _dtype_code(x2d), Q, d, int(decimal_places), bits, rebuild, wsptr, ws["bytes"],
                             kptr, klayout, keys.slice_weights.data_ptr(), keys.Sb, R,
                             _scale_inv(int(decimal_places), keys.decimals), R, _ptr(bias), out.data_ptr(), core, wptr,
                             wbytes, st), "bsi_hip_linear")
    _last_linear_rebuilt[0] = bool(rebuild)
    return out


def linear_cuda_forget() -> None:
    """Drop what linear_cuda remembers of its last build (and the input tensor it holds)."""
    for ws in _linear_ws.values():
        ws["capture"] = [None, None]
        for _, slot in ws["eager"].values():
            slot[0], slot[1] = None, None


def _dot_result(out, ns, Q, R):
    per_q = float(ns) / float(Q) if Q > 0 else 0.0
    per_s = float(ns) / (float(Q) * float(R)) if (Q > 0 and R > 0) else 0.0
    return out, int(ns), per_q, per_s


def batch_dot_product_multiquery_cuda_batch_caps(query_batch_cap, keyset_cuda_cap, bias=None, warm_keys=None):
    """bsi_cuda.cpp:658-815 -> (out[Q, R] float32 on the device, dot_ns_total, ns_per_query, ns_per_scalar).
    The times are zero unless BSI_PROFILE=1 (which synchronises), as in the reference.
    ``bias`` (not in the reference's signature): an optional float32 [R] device tensor added to every output
    row in the same launch, rounded as ``out + bias`` would be.  ``warm_keys`` (not in the reference either): the
    keyset the next dot will use; this launch also reads it once so that it is cache-resident by then."""
    keys = _capsule(keyset_cuda_cap, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule")
    if isinstance(query_batch_cap, PrebuiltBSIQueryBatchHybridCUDA):
        # the batched hybrid form: EWAH streams, decoded in the dot's load stage
        hb = query_batch_cap
        _check(hb.W == keys.W, "Word count mismatch between query batch and keys")
        _check(keys.num_keys > 0, "Empty keys")
        _check(hb.decimals == keys.decimals, f"Decimal mismatch between queries and keys: q={hb.decimals} k={keys.decimals}")
        if bias is not None:
            _check(bias.is_cuda and bias.dtype == torch.float32 and bias.dim() == 1 and bias.numel() == keys.num_keys
                   and bias.is_contiguous(), "bias must be a contiguous float32 CUDA tensor of [R]")
        out, ns = _dot_ewah_batch(hb, keys, bias=bias)
        return _dot_result(out, ns, hb.Q, keys.num_keys)
    qb = _capsule(query_batch_cap, PrebuiltBSIQueryBatchCUDA, "Invalid CUDA query-batch capsule")
    _check(qb.words is not None and qb.slice_weights is not None, "Query batch tensors are not defined")
    _check(qb.words.is_cuda and qb.slice_weights.is_cuda, "Query batch tensors must be CUDA tensors")
    _check(qb.words.dim() == 3, "Query batch words must be [Q, Sa, W]")
    _check(qb.slice_weights.dim() == 2, "Query batch slice_weights must be [Q, Sa]")
    Q, Sa, W = qb.words.shape
    _check(Q > 0 and Sa > 0 and W > 0, "Empty query batch")
    _check(W == keys.W, "Word count mismatch between query batch and keys")
    _check(tuple(qb.slice_weights.shape) == (Q, Sa), f"slice_weights shape mismatch: expected [{Q}, {Sa}]")
    R = keys.num_keys
    _check(R > 0, "Empty keys")
    have_chunk_scales = qb.chunk_scales is not None and qb.chunk_scales.numel() > 0
    if have_chunk_scales:
        _check(qb.chunk_scales.is_cuda, "chunk_scales must be a CUDA tensor")
        _check(qb.chunk_scales.dim() == 2, "Expected [Q, chunks] chunk scales")
        _check(qb.chunk_scales.shape[0] == Q, "chunk_scales Q mismatch")
        _check(keys.W % 4 == 0, "Chunk scales require W64 multiple of 4")
        _check(qb.chunk_scales.shape[1] == keys.W // 4,
               f"Chunk scale stride mismatch: got {qb.chunk_scales.shape[1]} expected {keys.W // 4}")
        scales, stride = qb.chunk_scales, int(qb.chunk_scales.shape[1])
    elif qb.fixed:
        _check(qb.row_scales is not None, "Query batch has neither chunk scales nor row scales")
        scales, stride = qb.row_scales, 1
    _check(qb.decimals == keys.decimals,
           f"Decimal mismatch between queries and keys: q={qb.decimals} k={keys.decimals}")
    if bias is not None:
        _check(bias.is_cuda and bias.dtype == torch.float32 and bias.dim() == 1 and bias.numel() == R and bias.is_contiguous(),
               "bias must be a contiguous float32 CUDA tensor of [R]")
    if qb.fixed and keys.fixed:
        if warm_keys is not None:
            _capsule(warm_keys, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule (warm_keys)")
        out, ns = _dot(qb.words, qb.ints8, scales, stride, int(Sa), int(W), keys, int(Q), qb.decimals, bias=bias,
                       warm_keys=warm_keys)
    else:
        # a decimal-mode operand on either side: its slice weights carry everything, per-chunk scales cannot apply
        _check(not have_chunk_scales, "chunk-scaled queries need fixed-bit keys (BSI_FIXED_BITS_KEYS > 0)")
        out, ns = _dot_weighted(qb.words, qb.slice_weights, int(Sa), int(W), keys, int(Q), qb.decimals, bias=bias,
                                q_digits=qb.digits8 if not qb.fixed else None,
                                q_image=qb.ints8 if qb.fixed else None)
    return _dot_result(out, ns, Q, R)


def batch_dot_product_multiquery_cuda_caps(query_caps_list, keyset_cuda_cap):
    """bsi_cuda.cpp:433-656: list-of-row-handles form; rows are stacked, then the same dot runs."""
    keys = _capsule(keyset_cuda_cap, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule")
    R = keys.num_keys
    Q = len(query_caps_list)
    _check(R > 0 and Q > 0, "Empty keys or queries")
    rows = []
    for qi, cap in enumerate(query_caps_list):
        _check(isinstance(cap, _Capsule), "Each item must be a capsule")
        q = _capsule(cap, PrebuiltBSIQueryCUDA, f"Invalid BSI query capsule at index {qi}")
        _check(q.W == keys.W, "Word count mismatch between query and keys")
        _check(q.decimals == rows[0].decimals if rows else True, "Decimal mismatch across queries not supported")
        _check(q.S == rows[0].S if rows else True, "Mixed slice counts across queries are not supported")
        rows.append(q)
    have_scales = rows[0].chunk_scales is not None and rows[0].chunk_scales.numel() > 0
    for q in rows:
        _check((q.chunk_scales is not None and q.chunk_scales.numel() > 0) == have_scales,
               "Mixed chunk-scale and non-chunk-scale queries in the same group")
    f = _flags()
    q0 = rows[0]
    if not (keys.fixed and all(q.fixed for q in rows)):
        _check(all(q.fixed == q0.fixed for q in rows), "Mixed fixed-bit and decimal queries in the same group")
        _check(not have_scales, "chunk-scaled queries need fixed-bit keys (BSI_FIXED_BITS_KEYS > 0)")
        _check(q0.decimals == keys.decimals, f"Decimal mismatch between queries and keys: q={q0.decimals} k={keys.decimals}")
        words = torch.stack([q.dev_words for q in rows]).contiguous()
        weights = torch.stack([q.slice_weights for q in rows]).contiguous()
        digits = None
        if not q0.fixed and all(q.digits8 is not None for q in rows):
            digits = torch.stack([q.digits8 for q in rows], dim=1).contiguous()
        out, ns = _dot_weighted(words, weights, q0.S, keys.W, keys, Q, q0.decimals, q_digits=digits)
        return _dot_result(out, ns, Q, R)
    if (Q == 1 and getattr(q0, "comp_words", None) is not None and q0.comp_words.numel() > 0 and f["ewah_inline"]
            and keys.layout == _lib.LAYOUT_TILED16 and keys.Sb == 6 and 2 <= q0.S <= 8
            and f["core"] != _lib.CORE_VALU and q0.S * ((keys.W + 3) // 4) * 32 <= 96 * 1024):
        # a hybrid query: its EWAH streams are decoded inside the dot's load stage
        _check(q0.decimals == keys.decimals, f"Decimal mismatch between queries and keys: q={q0.decimals} k={keys.decimals}")
        if have_scales:
            sc, stride = q0.chunk_scales.contiguous(), int(q0.chunk_scales.numel())
            _check(keys.W % 4 == 0 and stride == keys.W // 4, "Chunk scale stride mismatch")
        else:
            sc, stride = q0.row_scale.reshape(1).contiguous(), 1
        out = torch.empty((1, R), dtype=torch.float32, device=q0.comp_words.device)
        prof = f["profile"]
        if prof:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
        check(lib.bsi_hip_dot_ewah_query(q0.comp_words.data_ptr(), q0.comp_off.data_ptr(), q0.comp_len.data_ptr(),
                                         q0.S, keys.W, sc.data_ptr(), stride, keys.words.data_ptr(),
                                         keys.slice_weights.data_ptr(), keys.Sb, R, _scale_inv(q0.decimals, keys.decimals),
                                         out.data_ptr(), None, _stream()), "bsi_hip_dot_ewah_query")
        ns = 0
        if prof:
            e1.record()
            e1.synchronize()
            ns = int(e0.elapsed_time(e1) * 1.0e6)
        return _dot_result(out, ns, 1, R)
    words = torch.stack([q.dev_words for q in rows]).contiguous()
    if have_scales:
        scales = torch.stack([q.chunk_scales for q in rows]).contiguous()
        _check(keys.W % 4 == 0 and scales.shape[1] == keys.W // 4, "Chunk scale stride mismatch")
        stride = int(scales.shape[1])
    else:
        scales = torch.stack([q.row_scale.reshape(()) for q in rows]).contiguous()
        stride = 1
    ints8 = torch.stack([q.ints8 for q in rows]).contiguous() if all(q.ints8 is not None for q in rows) else None
    _check(rows[0].decimals == keys.decimals,
           f"Decimal mismatch between queries and keys: q={rows[0].decimals} k={keys.decimals}")
    out, ns = _dot(words, ints8, scales, stride, rows[0].S, keys.W, keys, Q, rows[0].decimals)
    return _dot_result(out, ns, Q, R)


def bsi_keys_cuda_stats(keyset_cuda_cap) -> dict:
    """bsi_cuda.cpp:817-832."""
    keys = _capsule(keyset_cuda_cap, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule")
    return {"W": keys.W, "d": keys.d, "num_keys": keys.num_keys, "decimals": keys.decimals,
            "threshold": keys.threshold, "Sb_counts": {keys.Sb: keys.num_keys}}


def bsi_query_caps_stats(query_caps_list) -> dict:
    """bsi_cuda.cpp:834-861."""
    Q = len(query_caps_list)
    _check(Q > 0, "Empty query capsule list")
    counts: dict = {}
    W = -1
    for qi, cap in enumerate(query_caps_list):
        _check(isinstance(cap, _Capsule), "Each item must be a capsule")
        q = _capsule(cap, PrebuiltBSIQueryCUDA, f"Invalid BSI query capsule at index {qi}")
        counts[q.S] = counts.get(q.S, 0) + 1
        if W < 0:
            W = q.W
        else:
            _check(q.W == W, "Word count mismatch across queries")
    return {"Q": Q, "W": W, "S_counts": counts}


# --------------------------------------------------------------------------- parity / debug hooks


def debug_chunk_ints(query_batch_cap, keyset_cuda_cap, core: str = "auto"):
    """Integer accumulators I[q, r, c] (int32) and the fp32 output of one dot, for parity checks.
    No counterpart in the reference (its accumulators never leave the kernel)."""
    keys = _capsule(keyset_cuda_cap, PrebuiltBSIKeysCUDA, "Invalid CUDA keys capsule")
    qb = _capsule(query_batch_cap, PrebuiltBSIQueryBatchCUDA, "Invalid CUDA query-batch capsule")
    _check(qb.fixed and keys.fixed, "debug_chunk_ints: per-chunk accumulators exist for fixed-bit operands only")
    Q, Sa, W = qb.words.shape
    chunks = (W + 3) // 4
    ints = torch.zeros((Q, keys.num_keys, chunks), dtype=torch.int32, device=qb.words.device)
    if qb.chunk_scales is not None and qb.chunk_scales.numel() > 0:
        scales, stride = qb.chunk_scales, int(qb.chunk_scales.shape[1])
    else:
        scales, stride = qb.row_scales, 1
    code = {"auto": _lib.CORE_AUTO, "valu": _lib.CORE_VALU, "mfma": _lib.CORE_MFMA}[core]
    out, _ = _dot(qb.words, qb.ints8, scales, stride, int(Sa), int(W), keys, int(Q), qb.decimals, chunk_ints=ints, core=code)
    return ints, out


def debug_quantize_int64_cpu(values: torch.Tensor, decimal_places: int) -> torch.Tensor:
    """bsiFunctions.cpp:760-774: round-half-away quantisation on the host (a CPU function in the
    reference too; exact for float inputs because the fp64 product and the +0.5 are exact)."""
    x = values.detach().to("cpu", torch.float32).to(torch.float64) * (10.0 ** int(decimal_places))
    return torch.where(x >= 0, torch.floor(x + 0.5), -torch.floor(-x + 0.5)).to(torch.int64)


# The reference's scalar ("non-CUDA") entry points (bsiFunctions.cpp:811-846): served by the device kernels here.
from .bsi_scalar import (  # noqa: E402,F401
    PrebuiltBSIKeys, PrebuiltBSIQuery, batch_dot_product, batch_dot_product_prebuilt, batch_dot_product_prebuilt_capsule,
    build_bsi_keys, build_bsi_query, debug_bsi_query_words, dot_product, dot_product_decimal, keyset_size_on_disk,
    keyset_slice_stats, random_number_dot_product_bsi, random_number_dot_product_vector, save_keyset, tensor_slice_stats,
    vector_dot_product, vector_dot_product_no_precison)
