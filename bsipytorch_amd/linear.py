"""``BSIQuantizedLinear``: the BSI-linear drop-in for ``torch.nn.Linear`` and the model-wide
replacement helper, mirroring ``bsi_ops/benchmarks/verify_accuracy_bsi.py:46-215,217-279,312-368,444-486``
of the reference (same constructor arguments, attributes, counters and scope rules).

forward(x): flatten to [Q, D] -> build query planes on the GPU -> BSI dot against the prebuilt key
planes -> cast to x.dtype -> add bias -> restore the leading shape.
"""
from __future__ import annotations

import json
import os
import time
from typing import Any, Dict, List, Union

import torch
import torch.nn as nn

from . import bsi_ops


# Layers fed by the same activation tensor (q_proj / k_proj / v_proj) share one query build: the last built
# batch is kept with a reference to its input (so its address cannot be reused) and its version counter.
_last_query_build: Dict[str, Any] = {}


def forget_shared_builds() -> None:
    """Drop every remembered query build (the shared build of sibling layers, the one-call path's workspaces).  Call it
    before and after recording a forward into a HIP graph: what was built while recording has not run, and what
    an earlier recording built is not part of a new graph."""
    _last_query_build.clear()
    bsi_ops.linear_cuda_forget()


def _cached_query_build(batch_inputs: torch.Tensor, decimal_places: int, threshold: float, packed: bool):
    use_cache = bsi_ops.fast_getenv("BSI_QUERY_CACHE", "1") != "0"
    # (the capture's identifier is part of the key: a build that one graph capture recorded is not part of another's)
    key = bsi_ops.tensor_build_key(batch_inputs, int(decimal_places), bool(packed), bsi_ops.capture_id()) if use_cache else None
    use_cache = use_cache and key is not None  # a tensor without a version counter (inference mode) is built anew
    if use_cache and _last_query_build.get("key") == key and _last_query_build.get("src") is not None:
        return _last_query_build["cap"], True
    if packed:
        cap = bsi_ops.build_bsi_queries_cuda_batch_packed(batch_inputs, decimal_places, threshold)
    else:
        cap = bsi_ops.build_bsi_queries_cuda_batch(batch_inputs, decimal_places, threshold)
    if use_cache:
        _last_query_build.update(key=key, src=batch_inputs, cap=cap)
    return cap, False


class BSIQuantizedLinear(nn.Module):
    """Linear layer whose weight lives as BSI key planes (verify_accuracy_bsi.py:46-215)."""

    def __init__(self, original_linear, decimalPlaces=2, compress_threshold=0.2, query_threshold=None,
                 prefer_cuda: bool = True, prebuilt_keys=None):
        super().__init__()
        self.decimalPlaces = int(decimalPlaces)
        self.compress_threshold = float(compress_threshold)
        self.query_compress_threshold = float(query_threshold) if query_threshold is not None else float(compress_threshold)
        self.in_features = original_linear.in_features
        self.out_features = original_linear.out_features

        if prebuilt_keys is not None:
            # keys read back from disk (load_bsi_model): the dense weight of `original_linear` is not looked at
            self.weight_fp32 = None
            self.weight_dense_memory_bytes = self.in_features * self.out_features * 4
            bias = original_linear.bias
            self.register_buffer("bias", None if bias is None else bias.detach().to(torch.float32))
            self.bias_fp32 = None if bias is None else self.bias.cpu()
            self.bias_memory_bytes = 0 if bias is None else self.bias.numel() * 4
            self._bsi_keys_cuda, total_mem_bytes, num_keys, d, _W = prebuilt_keys
            assert num_keys == self.out_features and d == self.in_features, "keyset does not fit this layer"
            assert self._bsi_keys_cuda.decimals == self.decimalPlaces, "keyset was built with other decimal places"
            self.weight_bsi_memory_bytes = int(total_mem_bytes)
            self.total_bsi_static_bytes = self.weight_bsi_memory_bytes + self.bias_memory_bytes
            self.verbose = False
            self.collect_stats = False
            self._reset_counters()
            return

        dense_weight = original_linear.weight.detach().to(torch.float32)
        self.weight_fp32 = dense_weight.cpu()
        self.weight_dense_memory_bytes = dense_weight.numel() * dense_weight.element_size()
        if original_linear.bias is not None:
            bias = original_linear.bias.detach().to(torch.float32)
            self.register_buffer("bias", bias)
            self.bias_fp32 = bias.cpu()
            self.bias_memory_bytes = bias.numel() * bias.element_size()
        else:
            self.register_buffer("bias", None)
            self.bias_fp32 = None
            self.bias_memory_bytes = 0

        assert prefer_cuda and torch.cuda.is_available(), \
            "CUDA path required: build_bsi_keys_cuda not available or CUDA not present"
        with torch.no_grad():
            # build from the tensor where it already lives: no host round trip for device weights
            src = dense_weight if dense_weight.is_cuda else self.weight_fp32
            self._bsi_keys_cuda, total_mem_bytes, num_keys, d, _W = bsi_ops.build_bsi_keys_cuda(
                src, self.decimalPlaces, float(self.compress_threshold))
        assert num_keys == self.out_features and d == self.in_features
        self.weight_bsi_memory_bytes = int(total_mem_bytes)
        self.total_bsi_static_bytes = self.weight_bsi_memory_bytes + self.bias_memory_bytes
        self.verbose = False
        self.collect_stats = False
        self._reset_counters()

    def _reset_counters(self):
        self.dot_ns_total = 0
        self.dot_calls = 0
        self.dot_kernel_ns_per_query_last = 0.0
        self.dot_kernel_ns_per_scalar_last = 0.0
        self.dot_query_vectors_total = 0
        self.dot_output_elements_total = 0
        self.build_ns_total = 0
        self.build_quantize_ns_total = 0
        self.build_pack_ns_total = 0
        self.build_kernel_ns_total = 0
        self.build_calls = 0

    def reset_error_stats(self):
        self.mse_sum = 0.0
        self.mae_sum = 0.0
        self.cosine_sum = 0.0
        self.max_abs_error = 0.0
        self.samples_tracked = 0

    def forward(self, x):
        original_dtype = x.dtype
        original_shape = x.shape
        if x.dim() != 2:
            x = x.reshape(-1, x.shape[-1])
        if bsi_ops.fast_getenv("BSI_QUERY_FP32", "0") != "0":
            x = x.to(torch.float32)
        batch_inputs = x.detach().contiguous()
        q_rows = int(batch_inputs.shape[0])

        # the counters live in the instance dict: nn.Module.__setattr__ costs more than the rest of this method
        c = self.__dict__
        if q_rows <= bsi_ops.FUSED_LINEAR_MAX_ROWS:
            scores = self._forward_few_rows(batch_inputs, original_dtype)
            if scores is not None:
                return scores.view(*original_shape[:-1], -1) if len(original_shape) != 2 else scores
        scores = self._forward_one_call(batch_inputs, original_dtype)
        if scores is not None:
            return scores.view(*original_shape[:-1], -1) if len(original_shape) != 2 else scores
        t0 = time.perf_counter_ns()
        use_packed = bsi_ops.fast_getenv("BSI_QUERY_PACKED", "1") != "0"
        qcap, reused = _cached_query_build(batch_inputs, self.decimalPlaces, float(self.query_compress_threshold),
                                           use_packed)
        c["build_ns_total"] += time.perf_counter_ns() - t0
        if not reused:
            q_ns, p_ns, t_ns = bsi_ops.get_last_query_build_profile_cuda()
            c["build_quantize_ns_total"] += int(q_ns)
            c["build_pack_ns_total"] += int(p_ns)
            c["build_kernel_ns_total"] += int(t_ns)
            c["build_calls"] += 1

        bias = self.bias
        # fp32 activations: the bias goes into the dot's epilogue (same rounding as scores + bias); in half
        # precision the reference adds it after the cast, so it stays a separate addition there
        fuse_bias = (use_packed and bias is not None and original_dtype == torch.float32 and bias.is_cuda
                     and bias.dtype == torch.float32 and bias.is_contiguous())
        fused = c.get("_fused") if use_packed else None
        if fused is not None:
            # this layer shares its input with siblings (q/k/v): one dot over their stacked keys serves all of them
            group, start, stop = fused
            all_scores, ns_total, ns_q, ns_s, bias_done = group.scores(qcap, fuse_bias)
            scores = all_scores[:, start:stop]
            fuse_bias = fuse_bias and bias_done
        elif use_packed:
            # the layer that runs next (set by quantize_model_bsi): its keys are touched by this dot's kernel so
            # that they are cache-resident when their turn comes
            nxt = c.get("_next_bsi_layer")
            scores, ns_total, ns_q, ns_s = bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(
                qcap, self._bsi_keys_cuda, bias if fuse_bias else None, _keys_to_warm(nxt))
        else:
            scores, ns_total, ns_q, ns_s = bsi_ops.batch_dot_product_multiquery_cuda_caps(qcap, self._bsi_keys_cuda)
        c["dot_kernel_ns_per_query_last"] = float(ns_q)
        c["dot_kernel_ns_per_scalar_last"] = float(ns_s)
        c["dot_query_vectors_total"] += q_rows
        c["dot_output_elements_total"] += q_rows * int(self.out_features)
        c["dot_ns_total"] += int(ns_total)
        c["dot_calls"] += 1

        if scores.dtype != original_dtype:
            scores = scores.to(dtype=original_dtype)
        if bias is not None and not fuse_bias:
            if bias.dtype != original_dtype or bias.device != scores.device:
                bias = bias.to(device=scores.device, dtype=original_dtype)
            scores = scores + bias
        if c.get("collect_stats") and self.weight_fp32 is not None:
            self._track_error(batch_inputs, scores)
        if len(original_shape) != 2:
            scores = scores.view(*original_shape[:-1], -1)
        return scores

    def _forward_one_call(self, batch_inputs, original_dtype):
        """Query build and dot in one library call (bsi_ops.linear_cuda), or None when that path does not serve the
        call: the same two launches as below with a fraction of the host work, which is what an eager forward of
        many small layers is bound by.  Layers fed the same tensor share the build (the workspace remembers what it
        was built from); fused q/k/v siblings share the whole call."""
        c = self.__dict__
        fused = c.get("_fused")
        keys = fused[0].keys if fused is not None else self._bsi_keys_cuda
        if (c.get("collect_stats") or bsi_ops.fast_getenv("BSI_QUERY_PACKED", "1") == "0" or bsi_ops.fast_getenv("BSI_QUERY_CACHE", "1") == "0"
                or not bsi_ops.can_linear_one_call(batch_inputs, keys)):
            return None
        fp32 = original_dtype == torch.float32
        if fused is not None:
            group, start, stop = fused
            key = bsi_ops.tensor_build_key(batch_inputs, bsi_ops.capture_id())
            last = group.__dict__.get("_last_call")
            if last is not None and key is not None and last[0] == key:
                scores, bias_done = last[2][:, start:stop], last[3]
                last[4] -= 1
                if last[4] <= 0:
                    group.__dict__["_last_call"] = None
            else:
                gb = bsi_ops.device_bias(group.bias, batch_inputs.device) if fp32 else None
                all_scores = bsi_ops.linear_cuda(batch_inputs, keys, self.decimalPlaces, gb, _keys_to_warm(group.next_layer), True)
                group.__dict__["_last_call"] = [key, batch_inputs, all_scores, gb is not None, len(group.members) - 1]
                scores, bias_done = all_scores[:, start:stop], gb is not None
                c["dot_calls"] += 1
                c["build_calls"] += int(bsi_ops._last_linear_rebuilt[0])
        else:
            b = bsi_ops.device_bias(self.bias, batch_inputs.device) if fp32 else None
            scores = bsi_ops.linear_cuda(batch_inputs, keys, self.decimalPlaces, b, _keys_to_warm(c.get("_next_bsi_layer")), True)
            bias_done = b is not None
            c["dot_calls"] += 1
            c["build_calls"] += int(bsi_ops._last_linear_rebuilt[0])
        q_rows = int(batch_inputs.shape[0])
        c["dot_query_vectors_total"] += q_rows
        c["dot_output_elements_total"] += q_rows * int(self.out_features)
        if scores.dtype != original_dtype:
            scores = scores.to(dtype=original_dtype)
        if self.bias is not None and not bias_done:
            scores = scores + self.bias.to(device=scores.device, dtype=original_dtype)
        return scores

    def _forward_few_rows(self, batch_inputs, original_dtype):
        """A decode step (at most 4 rows): query build and dot in one launch, or None when that kernel does not
        serve the call.  Siblings that share their input (fused q/k/v) share the launch."""
        c = self.__dict__
        fused = c.get("_fused")
        keys = fused[0].keys if fused is not None else self._bsi_keys_cuda
        if c.get("collect_stats") or not bsi_ops.can_fuse_linear_few_rows(batch_inputs, keys):
            return None
        # The fused kernel saves the host a launch and the handles of a query build, which is what an eager decode
        # step is bound by.  On the GPU it costs no more than the dot alone as long as every workgroup can request
        # its share of the activations before its key planes; past that (more rows, longer rows) it repeats too much
        # arithmetic, so a forward that is being captured into a graph, where host time does not count, then keeps
        # the two launches.  BSI_FUSED_LINEAR=2 forces the fused kernel in both cases.
        if (torch.cuda.is_current_stream_capturing() and bsi_ops.fast_getenv("BSI_FUSED_LINEAR", "1") != "2"
                and not bsi_ops.linear_few_rows_is_free(batch_inputs, keys)):
            return None
        fp32 = original_dtype == torch.float32
        bsi_ops.warm_query_build_caches(int(batch_inputs.shape[0]))
        bsi_ops.reserve_linear_workspace(batch_inputs)  # a later capture of this forward may take the one-call path
        if fused is not None:
            group, start, stop = fused
            key = bsi_ops.tensor_build_key(batch_inputs, bsi_ops.capture_id())
            last = group.__dict__.get("_last_few")
            if last is not None and key is not None and last[0] == key:
                scores, bias_done = last[2][:, start:stop], last[3]
                last[4] -= 1
                if last[4] <= 0:
                    group.__dict__["_last_few"] = None
            else:
                gb = bsi_ops.device_bias(group.bias, batch_inputs.device) if fp32 else None
                all_scores = bsi_ops.linear_few_rows_cuda(batch_inputs, keys, self.decimalPlaces, gb, True)
                # holds the input's storage (so that its address is not reused) until every member has been served
                group.__dict__["_last_few"] = [key, batch_inputs, all_scores, gb is not None, len(group.members) - 1]
                scores, bias_done = all_scores[:, start:stop], gb is not None
                c["dot_calls"] += 1
        else:
            b = bsi_ops.device_bias(self.bias, batch_inputs.device) if fp32 else None
            scores, bias_done = bsi_ops.linear_few_rows_cuda(batch_inputs, keys, self.decimalPlaces, b, True), b is not None
            c["dot_calls"] += 1
        q_rows = int(batch_inputs.shape[0])
        c["dot_query_vectors_total"] += q_rows
        c["dot_output_elements_total"] += q_rows * int(self.out_features)
        if scores.dtype != original_dtype:
            scores = scores.to(dtype=original_dtype)
        if self.bias is not None and not bias_done:
            scores = scores + self.bias.to(device=scores.device, dtype=original_dtype)
        return scores

    @torch.no_grad()
    def _track_error(self, batch_inputs, scores):
        """Error of this forward against the dense fp32 layer, accumulated per sample (row)."""
        w = self.weight_fp32.to(batch_inputs.device)
        ref = batch_inputs.to(torch.float32) @ w.t()
        if self.bias is not None:
            ref = ref + self.bias.to(torch.float32)
        got = scores.to(torch.float32)
        err = got - ref
        n = int(ref.shape[0])
        c = self.__dict__
        if "samples_tracked" not in c:
            self.reset_error_stats()
        c["mse_sum"] += float(err.pow(2).mean(dim=1).sum())
        c["mae_sum"] += float(err.abs().mean(dim=1).sum())
        c["cosine_sum"] += float(torch.nn.functional.cosine_similarity(got, ref, dim=1).sum())
        c["max_abs_error"] = max(c["max_abs_error"], float(err.abs().max()))
        c["samples_tracked"] += n


def _keys_to_warm(layer):
    """The keyset a dot should warm for `layer` (the whole stacked keyset when that layer is part of a fused group)."""
    if layer is None:
        return None
    fused = layer.__dict__.get("_fused")
    return fused[0].keys if fused is not None else layer._bsi_keys_cuda


class _FusedSiblings:
    """Layers fed by the same activation tensor (q_proj / k_proj / v_proj), served by ONE dot over their stacked
    keys; each member takes its columns of the result.  The result is kept for the query build it was computed
    from (the members share one build per input), so the first member called does the work."""

    def __init__(self, members):
        self.members = list(members)
        self.keys = bsi_ops.concat_keysets([m._bsi_keys_cuda for m in self.members])
        biases = [m.bias for m in self.members]
        self.bias = torch.cat([b.to(torch.float32) for b in biases]).contiguous() if all(b is not None for b in biases) else None
        self.next_layer = None
        self._last = None

    def scores(self, qcap, want_bias):
        """(scores of all members [Q, sum of out_features], dot times, whether the bias is already added)."""
        last = self._last
        if last is not None and last[0] is qcap:  # siblings share one query build: the same handle means the same input
            out, bias_done = last[1], last[2]
            last[3] -= 1
            if last[3] <= 0:  # every member has had its columns: nothing is held until the next forward
                self._last = None
            return out, 0, 0.0, 0.0, bias_done
        gb = bsi_ops.device_bias(self.bias, self.keys.words.device) if want_bias else None
        bias_done = gb is not None
        out, ns_total, ns_q, ns_s = bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(
            qcap, self.keys, gb, _keys_to_warm(self.next_layer))
        self._last = [qcap, out, bias_done, len(self.members) - 1]
        return out, ns_total, ns_q, ns_s, bias_done


def fuse_sibling_layers(model: nn.Module, names=("q_proj", "k_proj", "v_proj")) -> int:
    """Stack the keys of BSI layers that are children of one module under the given names (the attention
    projections, which read the same activations) so that one dot serves them all: three launches over 2048 key
    rows each become one over 6144, which fills the GPU with the large tile.  Every output element is computed
    from the same query row and key row as before, so the results are bit-identical.  The members' own keysets
    become views into the stacked one.  Returns the number of groups formed.  Not in the reference."""
    groups = 0
    for parent in model.modules():
        kids = [getattr(parent, n, None) for n in names]
        if not all(isinstance(k, BSIQuantizedLinear) for k in kids) or any(k.__dict__.get("_fused") for k in kids):
            continue
        k0 = kids[0]
        if any((k.in_features, k.decimalPlaces) != (k0.in_features, k0.decimalPlaces) or not k._bsi_keys_cuda.fixed
               or k.out_features % 64 != 0 for k in kids):
            continue
        group = _FusedSiblings(kids)
        start = 0
        for k in kids:
            k.__dict__["_fused"] = (group, start, start + k.out_features)
            k._bsi_keys_cuda = bsi_ops.keyset_rows(group.keys, start, start + k.out_features)
            start += k.out_features
        groups += 1
    link_bsi_layers(model)
    return groups


_COUNTERS = ("dot_ns_total", "dot_calls", "build_ns_total", "build_quantize_ns_total", "build_pack_ns_total",
             "build_kernel_ns_total", "build_calls", "dot_query_vectors_total", "dot_output_elements_total")


def reset_bsi_dot_counters(model: nn.Module):
    for m in model.modules():
        if isinstance(m, BSIQuantizedLinear):
            for c in _COUNTERS:
                setattr(m, c, 0)


def _sum(model: nn.Module, attr: str) -> int:
    return sum(int(getattr(m, attr, 0)) for m in model.modules() if isinstance(m, BSIQuantizedLinear))


def sum_bsi_dot_counters(model): return _sum(model, "dot_ns_total")
def sum_bsi_build_counters(model): return _sum(model, "build_ns_total")
def sum_bsi_build_quantize_counters(model): return _sum(model, "build_quantize_ns_total")
def sum_bsi_build_pack_counters(model): return _sum(model, "build_pack_ns_total")
def sum_bsi_build_kernel_counters(model): return _sum(model, "build_kernel_ns_total")
def sum_bsi_dot_query_vectors(model): return _sum(model, "dot_query_vectors_total")
def sum_bsi_dot_output_elements(model): return _sum(model, "dot_output_elements_total")


def summarize_bsi_model(model: nn.Module) -> Dict[str, Any]:
    """Per-layer and total byte accounting (verify_accuracy_bsi.py:312-368)."""
    s: Dict[str, Any] = dict(total_bsi_bytes=0, total_dense_bytes=0, total_bias_bytes=0, total_fp16_linear_bytes=0,
                             total_static_bytes=0, total_dense_with_bias_bytes=0, num_quantized_layers=0,
                             total_slices=0, compressed_slices=0, verbatim_slices=0, layers=[])
    for name, m in model.named_modules():
        if not isinstance(m, BSIQuantizedLinear):
            continue
        fp16_bytes = int(m.in_features * m.out_features * 2)
        s["layers"].append(dict(name=name, in_features=m.in_features, out_features=m.out_features,
                                decimalPlaces=m.decimalPlaces, compress_threshold=m.compress_threshold,
                                weight_bsi_bytes=m.weight_bsi_memory_bytes, weight_dense_bytes=m.weight_dense_memory_bytes,
                                bias_bytes=m.bias_memory_bytes, weight_fp16_bytes=fp16_bytes))
        # device keysets hold every slice verbatim (EWAH is applied to hybrid queries only)
        keys = m._bsi_keys_cuda
        slices = int(keys.num_keys * keys.Sb)
        disk = int(bsi_ops.keyset_size_on_disk_cuda(keys)[1])
        s["layers"][-1].update(weight_total_slices=slices, weight_verbatim_slices=slices, weight_compressed_slices=0,
                               weight_compressed_pct=0.0, weight_verbatim_pct=100.0 if slices else 0.0,
                               weight_bsi_disk_bytes=disk)
        s["total_slices"] += slices
        s["verbatim_slices"] += slices
        s["total_bsi_disk_bytes"] = s.get("total_bsi_disk_bytes", 0) + disk
        s["total_bsi_bytes"] += m.weight_bsi_memory_bytes
        s["total_dense_bytes"] += m.weight_dense_memory_bytes
        s["total_bias_bytes"] += m.bias_memory_bytes
        s["total_fp16_linear_bytes"] += fp16_bytes
        s["num_quantized_layers"] += 1
    s["total_static_bytes"] = s["total_bsi_bytes"] + s["total_bias_bytes"]
    s["total_dense_with_bias_bytes"] = s["total_dense_bytes"] + s["total_bias_bytes"]
    s["compressed_pct"] = 0.0
    s["verbatim_pct"] = 100.0 if s["total_slices"] else 0.0
    return s


def enable_bsi_error_stats(model: nn.Module, enabled: bool) -> None:
    """Toggle per-layer error tracking (verify_accuracy_bsi.py:282-290).  While it is on, every forward of a BSI
    layer also computes the dense fp32 result from the kept weights and accumulates MSE, MAE, cosine similarity
    and the largest absolute error (a debugging mode: it costs a dense matmul per layer)."""
    for module in model.modules():
        if isinstance(module, BSIQuantizedLinear):
            if enabled and not module.collect_stats:
                module.collect_stats = True
                module.reset_error_stats()
            elif not enabled:
                module.collect_stats = False


def collect_bsi_error_stats(model: nn.Module) -> List[Dict[str, float]]:
    """Accumulated per-layer error metrics, worst MSE first (verify_accuracy_bsi.py:293-310)."""
    out: List[Dict[str, float]] = []
    for name, m in model.named_modules():
        if isinstance(m, BSIQuantizedLinear) and getattr(m, "samples_tracked", 0) > 0:
            n = float(m.samples_tracked)
            out.append({"name": name, "decimalPlaces": m.decimalPlaces, "compress_threshold": m.compress_threshold,
                        "samples_tracked": n, "mse": m.mse_sum / n, "mae": m.mae_sum / n, "cosine": m.cosine_sum / n,
                        "max_abs": m.max_abs_error})
    out.sort(key=lambda item: item["mse"], reverse=True)
    return out


def get_model_static_bytes(model: nn.Module) -> int:
    """Parameters plus buffers, in bytes (benchmark_performance_bsi.py:488-492)."""
    return int(sum(p.nelement() * p.element_size() for p in model.parameters())
               + sum(b.nelement() * b.element_size() for b in model.buffers()))


def bsi_full_model_static_bytes(model: nn.Module, summary: Dict[str, Any]) -> int:
    """Static size of a BSI-quantised model: parameters and buffers (the non-BSI modules and the BSI biases) plus
    the BSI key bytes, which are not parameters (verify_accuracy_bsi.py:389-402)."""
    return get_model_static_bytes(model) + int(summary.get("total_bsi_bytes", 0))


def compression_summary_lines(summary: Dict[str, Any]):
    """(one line per layer, (compressed slices, all slices, percentage)) -- verify_accuracy_bsi.py:405-418."""
    lines = []
    for idx, layer in enumerate(summary.get("layers", []), start=1):
        total = int(layer.get("weight_total_slices", 0) or 0)
        compressed = int(layer.get("weight_compressed_slices", 0) or 0)
        pct = (compressed * 100.0 / total) if total else 0.0
        lines.append(f"Layer {idx} ({layer.get('name', f'Layer {idx}')}): {compressed}/{total} ({pct:.2f}%)")
    total = int(summary.get("total_slices", 0) or 0)
    compressed = int(summary.get("compressed_slices", 0) or 0)
    return lines, (compressed, total, (compressed * 100.0 / total) if total else 0.0)


def print_compression_summary(summary: Dict[str, Any], heading: str = "Compression Summary") -> None:
    """verify_accuracy_bsi.py:421-432."""
    lines, (compressed, total, pct) = compression_summary_lines(summary)
    print(f"\n=== {heading} ===")
    if not lines and total == 0:
        print("No compression statistics available.")
        return
    for line in lines:
        print(line)
    print(f"Overall compressed slices: {compressed}/{total} ({pct:.2f}%)")


def build_layer_config(default_value, attention_value, mlp_value):
    """Per-scope configuration for quantize_model_bsi (benchmark_performance_bsi.py:494-503)."""
    if attention_value is None and mlp_value is None:
        return default_value
    config = {"default": default_value}
    if attention_value is not None:
        config["attention"] = attention_value
    if mlp_value is not None:
        config["mlp"] = mlp_value
    return config


def _resolve_layer_value(config: Union[float, Dict[str, float]], layer_kind: str, fallback: float) -> float:
    if isinstance(config, dict):
        if layer_kind in ("attention", "mlp"):
            return float(config.get(layer_kind, config.get("default", fallback)))
        return float(config.get("default", fallback))
    return float(config)


_ATTN_TOKENS = ("attn", "self_attn", "q_proj", "k_proj", "v_proj", "out_proj")
_MLP_TOKENS = ("mlp", "ff", "ffn", "fc1", "fc2")


def quantize_model_bsi(model, decimalPlaces=2, skip_lm_head=True, scope="all", compress_threshold=0.2,
                       prefer_cuda: bool = True, verbose: bool = True, fuse_qkv: bool = False):
    """Replace every ``nn.Linear`` (except ``lm_head``) by ``BSIQuantizedLinear``; ``scope`` is
    'all' | 'attention' | 'mlp', chosen by name tokens (verify_accuracy_bsi.py:444-486)."""
    default_decimal = float(decimalPlaces if isinstance(decimalPlaces, (int, float)) else decimalPlaces.get("default", 2))
    default_threshold = float(compress_threshold if isinstance(compress_threshold, (int, float))
                              else compress_threshold.get("default", 0.2))
    targets: List[str] = []
    for name, module in model.named_modules():
        if not isinstance(module, nn.Linear):
            continue
        if skip_lm_head and "lm_head" in name:
            continue
        is_attn = any(t in name for t in _ATTN_TOKENS)
        is_mlp = any(t in name for t in _MLP_TOKENS)
        if scope == "attention" and not is_attn:
            continue
        if scope == "mlp" and not is_mlp:
            continue
        targets.append(name)
    for name in targets:
        parent = model
        parts = name.split(".")
        for part in parts[:-1]:
            parent = getattr(parent, part)
        module = getattr(parent, parts[-1])
        kind = "attention" if any(t in name for t in _ATTN_TOKENS) else "mlp" if any(t in name for t in _MLP_TOKENS) else "other"
        setattr(parent, parts[-1], BSIQuantizedLinear(
            module, decimalPlaces=_resolve_layer_value(decimalPlaces, kind, default_decimal),
            compress_threshold=_resolve_layer_value(compress_threshold, kind, default_threshold),
            prefer_cuda=prefer_cuda))
    link_bsi_layers(model)
    if fuse_qkv:  # not in the reference's signature: see fuse_sibling_layers
        fuse_sibling_layers(model)
    if verbose:
        print(f"Quantized {len(targets)} linear layers to BSI with decimalPlaces={decimalPlaces} (scope={scope})")
    return model


def link_bsi_layers(model: nn.Module) -> int:
    """Tell every BSI layer which one runs after it (module order, the last one wrapping round to the first), so
    that its dot can warm the cache with the next layer's keys: in a model every keyset has been evicted by the
    time its layer comes round again, and the dot kernel runs 15-35 % slower on keys that come from HBM.
    ``BSI_WARM_NEXT=0`` leaves the layers unlinked.  Returns the number of layers linked."""
    layers = [m for m in model.modules() if isinstance(m, BSIQuantizedLinear)]
    on = os.getenv("BSI_WARM_NEXT", "1") != "0" and len(layers) > 1
    for i, m in enumerate(layers):
        m.__dict__["_next_bsi_layer"] = layers[(i + 1) % len(layers)] if on else None
    for i, m in enumerate(layers):  # a fused group warms the first layer after its last member
        fused = m.__dict__.get("_fused")
        if fused is not None and m is fused[0].members[-1]:
            nxt = m.__dict__["_next_bsi_layer"]
            fused[0].next_layer = nxt if (nxt is not None and nxt.__dict__.get("_fused", (None,))[0] is not fused[0]) else None
    return len(layers) if on else 0


class GraphedForward:
    """``model(*inputs)`` recorded once into a HIP graph and replayed: the whole forward becomes one submission with no
    host work per layer (an eager forward of many small BSI layers is bound by that work).  Not in the reference.

    ``example_inputs`` fix the shapes and dtypes; a call copies its inputs into the recorded input tensors, replays the
    graph and returns the recorded output object (whatever the model returns), whose tensors are overwritten by the
    next call.  Eager forwards of the same model may run in between.  The model must not change between calls in ways
    a recording cannot see (weights rebuilt, layers swapped, environment flags): record again then."""

    def __init__(self, model: nn.Module, *example_inputs: torch.Tensor, warmup: int = 2):
        if not torch.cuda.is_available():
            raise RuntimeError("GraphedForward needs the GPU")
        if not example_inputs or not all(isinstance(t, torch.Tensor) and t.is_cuda for t in example_inputs):
            raise ValueError("GraphedForward takes device tensors as example inputs")
        if bsi_ops._flags()["profile"]:
            raise RuntimeError("BSI_PROFILE=1 times every dot with events and synchronises: that cannot be recorded into a graph")
        if bsi_ops._flags()["bits_q"] == 0:
            raise RuntimeError("decimal-mode query builds (BSI_FIXED_BITS*=0) read their slice count back from the device, "
                               "as the reference's do: that cannot be recorded into a graph")
        self.model = model
        self.static_inputs = [t.clone() for t in example_inputs]
        with torch.no_grad():
            # warm-up on a side stream, as captures need: allocates every workspace and key layout the forward uses
            forget_shared_builds()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(max(1, int(warmup))):
                    model(*self.static_inputs)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            forget_shared_builds()
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self.static_output = model(*self.static_inputs)
            forget_shared_builds()

    def __call__(self, *inputs: torch.Tensor):
        if len(inputs) != len(self.static_inputs):
            raise ValueError(f"recorded with {len(self.static_inputs)} inputs, called with {len(inputs)}")
        for static, t in zip(self.static_inputs, inputs):
            if t.shape != static.shape or t.dtype != static.dtype:
                raise ValueError(f"recorded for inputs of shape {tuple(static.shape)} and dtype {static.dtype}, "
                                 f"called with {tuple(t.shape)} {t.dtype}")
            if t.data_ptr() != static.data_ptr():
                static.copy_(t)
        self.graph.replay()
        return self.static_output


def save_bsi_model(model: nn.Module, out_dir: str) -> List[Dict[str, Any]]:
    """Write every BSI layer's keyset (and bias) under ``out_dir`` with a ``manifest.json`` holding the fields the
    reference's save_bsi_model records (verify_accuracy_bsi.py:370-386: name, in, out, decimalPlaces,
    compress_threshold) plus the file sizes.  One ``keyset.bsik`` per layer instead of one file per key and slice."""
    os.makedirs(out_dir, exist_ok=True)
    meta = []
    for name, module in model.named_modules():
        if not isinstance(module, BSIQuantizedLinear):
            continue
        layer_dir = os.path.join(out_dir, name.replace(".", "_"))
        nbytes = bsi_ops.save_keyset_cuda(module._bsi_keys_cuda, layer_dir)
        if module.bias is not None:
            with open(os.path.join(layer_dir, "bias.f32"), "wb") as fh:
                fh.write(module.bias.detach().cpu().numpy().astype("<f4", copy=False).tobytes())
        meta.append({"name": name, "in": module.in_features, "out": module.out_features,
                     "decimalPlaces": module.decimalPlaces, "compress_threshold": module.compress_threshold,
                     "dir": os.path.basename(layer_dir), "keyset_bytes": int(nbytes), "has_bias": module.bias is not None})
    with open(os.path.join(out_dir, "manifest.json"), "w") as f:
        json.dump(meta, f, indent=2)
    return meta


def load_bsi_model(model: nn.Module, out_dir: str, verbose: bool = False) -> nn.Module:
    """Replace the ``nn.Linear`` layers named in ``out_dir/manifest.json`` by BSI layers whose keys (and bias) are
    read from disk: no re-quantisation, and the dense weights of ``model`` are never read for those layers."""
    import numpy as np

    with open(os.path.join(out_dir, "manifest.json")) as f:
        meta = json.load(f)
    for entry in meta:
        parent = model
        parts = entry["name"].split(".")
        for part in parts[:-1]:
            parent = getattr(parent, part)
        module = getattr(parent, parts[-1])
        assert (module.in_features, module.out_features) == (entry["in"], entry["out"]), \
            f"{entry['name']}: layer shape differs from the saved keyset"
        layer_dir = os.path.join(out_dir, entry["dir"])
        shell = nn.Linear(entry["in"], entry["out"], bias=entry["has_bias"], device="meta")
        if entry["has_bias"]:
            b = np.fromfile(os.path.join(layer_dir, "bias.f32"), dtype="<f4")
            assert b.size == entry["out"], f"{entry['name']}: truncated bias file"
            shell.bias = nn.Parameter(torch.from_numpy(b).cuda(), requires_grad=False)
        setattr(parent, parts[-1], BSIQuantizedLinear(
            shell, decimalPlaces=entry["decimalPlaces"], compress_threshold=entry["compress_threshold"],
            prebuilt_keys=bsi_ops.load_keyset_cuda(layer_dir)))
    link_bsi_layers(model)
    if verbose:
        print(f"Loaded {len(meta)} BSI layers from {out_dir}")
    return model
