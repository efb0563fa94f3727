"""OPT-architecture prefill with every decoder linear layer replaced by the BSI-linear drop-in.

Counterpart of the timing legs of ``bsi_ops/benchmarks/benchmark_performance_bsi.py:143-396`` of the
reference (forward ms by device events, build/dot ms from the per-layer counters), without the parts
that need the network: weights are random ~N(0, 0.02) on the OPT architecture named by ``--model``,
token ids are uniform random from a seed, and no accuracy is computed.

    python -m bsipytorch_amd.benchmarks.benchmark_opt_prefill --model opt-1.3b --seq_len 512

Reports tokens/s of one prefill (batch 1), run eagerly and as a replayed HIP graph, the share of
the forward spent in the BSI dot kernels (device-event time per call, collected in a second pass with BSI_PROFILE=1 because per-call events
synchronise), the query-build time, and the dense fp32 forward of the same model for context.
"""
from __future__ import annotations

import argparse
import json
import os
import time

import torch
import torch.nn as nn
import torch.nn.functional as F

SHAPES = {
    # name: (layers, hidden, heads, ffn, vocab)
    "opt-125m": (12, 768, 12, 3072, 50272),
    "opt-350m-shape": (24, 1024, 16, 4096, 50272),
    "opt-1.3b": (24, 2048, 32, 8192, 50272),
    "opt-2.7b": (32, 2560, 32, 10240, 50272),
    "opt-6.7b": (32, 4096, 32, 16384, 50272),
}


class OPTAttention(nn.Module):
    def __init__(self, hidden, heads):
        super().__init__()
        self.heads, self.head_dim = heads, hidden // heads
        self.q_proj = nn.Linear(hidden, hidden)
        self.k_proj = nn.Linear(hidden, hidden)
        self.v_proj = nn.Linear(hidden, hidden)
        self.out_proj = nn.Linear(hidden, hidden)

    def forward(self, x):
        b, t, h = x.shape
        shp = (b, t, self.heads, self.head_dim)
        q = self.q_proj(x).view(shp).transpose(1, 2)
        k = self.k_proj(x).view(shp).transpose(1, 2)
        v = self.v_proj(x).view(shp).transpose(1, 2)
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        return self.out_proj(a.transpose(1, 2).reshape(b, t, h))


class OPTDecoderLayer(nn.Module):
    """Pre-layer-norm decoder block: LN -> self-attention -> +x ; LN -> fc1 -> ReLU -> fc2 -> +x."""

    def __init__(self, hidden, heads, ffn):
        super().__init__()
        self.self_attn = OPTAttention(hidden, heads)
        self.self_attn_layer_norm = nn.LayerNorm(hidden)
        self.fc1 = nn.Linear(hidden, ffn)
        self.fc2 = nn.Linear(ffn, hidden)
        self.final_layer_norm = nn.LayerNorm(hidden)

    def forward(self, x):
        x = x + self.self_attn(self.self_attn_layer_norm(x))
        return x + self.fc2(F.relu(self.fc1(self.final_layer_norm(x))))


class OPTModel(nn.Module):
    def __init__(self, layers, hidden, heads, ffn, vocab, max_pos=2048):
        super().__init__()
        self.embed_tokens = nn.Embedding(vocab, hidden)
        self.embed_positions = nn.Embedding(max_pos + 2, hidden)  # OPT offsets positions by 2
        self.layers = nn.ModuleList([OPTDecoderLayer(hidden, heads, ffn) for _ in range(layers)])
        self.final_layer_norm = nn.LayerNorm(hidden)
        self.lm_head = nn.Linear(hidden, vocab, bias=False)

    def forward(self, input_ids):
        pos = torch.arange(input_ids.shape[1], device=input_ids.device) + 2
        x = self.embed_tokens(input_ids) + self.embed_positions(pos)[None]
        for layer in self.layers:
            x = layer(x)
        return self.lm_head(self.final_layer_norm(x))


def build_model(name: str, seed: int, device: str) -> OPTModel:
    layers, hidden, heads, ffn, vocab = SHAPES[name]
    with torch.device(device):
        model = OPTModel(layers, hidden, heads, ffn, vocab)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    with torch.no_grad():
        for n, p in model.named_parameters():
            if "layer_norm" in n:
                continue
            if n.endswith("bias"):
                p.zero_()
            else:
                p.normal_(0.0, 0.02, generator=gen)
    return model.eval()


@torch.no_grad()
def time_forward(model, input_ids, iters: int, warmup: int):
    for _ in range(warmup):
        model(input_ids)
    torch.cuda.synchronize()
    times = []
    for _ in range(iters):
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        model(input_ids)
        e.record()
        torch.cuda.synchronize()
        times.append(s.elapsed_time(e))
    times.sort()
    return times[len(times) // 2], times[0]


@torch.no_grad()
def kernel_time_of_dots_and_builds(model, input_ids, replays: int = 5):
    """(dot ms, query-build ms) per forward as GPU time without any synchronisation in between: every BSI layer's dot
    -- on the activations the layer sees in this forward, with its bias and its warm-up of the next keyset as the
    forward launches it -- recorded into one HIP graph and replayed, and the query builds likewise (layers fed the
    same tensor share one build, as in the forward).  Per-call device events (BSI_PROFILE=1) synchronise after every
    call and so charge each dot its launch latency as well; these figures do not."""
    from bsipytorch_amd import bsi_ops, linear

    layers = [m for m in model.modules() if isinstance(m, linear.BSIQuantizedLinear)]
    seen = {}

    def note_input(mod, args):
        seen[id(mod)] = args[0]  # kept alive, so that no later tensor takes its address

    hooks = [m.register_forward_pre_hook(note_input) for m in layers]
    model(input_ids)
    for h in hooks:
        h.remove()
    builds, dots, groups_done, prev = [], [], set(), None
    for m in layers:
        x = seen[id(m)]
        x2d = x.reshape(-1, x.shape[-1]).detach().contiguous()
        fused = m.__dict__.get("_fused")
        if fused is not None:
            group = fused[0]
            if id(group) in groups_done:
                continue
            groups_done.add(id(group))
            keys, bias, nxt = group.keys, group.bias, group.next_layer
        else:
            keys, bias, nxt = m._bsi_keys_cuda, m.bias, m.__dict__.get("_next_bsi_layer")
        thr = float(m.query_compress_threshold)
        if x is not prev:
            builds.append(lambda x2d=x2d, dec=m.decimalPlaces, thr=thr: bsi_ops.build_bsi_queries_cuda_batch_packed(x2d, dec, thr))
        prev = x
        qcap = bsi_ops.build_bsi_queries_cuda_batch_packed(x2d, m.decimalPlaces, thr)
        b = bsi_ops.device_bias(bias, x2d.device) if (bias is not None and x.dtype == torch.float32) else None
        dots.append(lambda q=qcap, k=keys, b=b, w=linear._keys_to_warm(nxt):
                    bsi_ops.batch_dot_product_multiquery_cuda_batch_caps(q, k, b, w))

    def replayed_ms(launches):
        for f in launches:  # once eagerly: workspaces and scratch regions exist before the capture
            f()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            kept = [f() for f in launches]  # the outputs stay allocated while the graph lives
        times = []
        for _ in range(replays + 1):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            g.replay()
            e.record()
            torch.cuda.synchronize()
            times.append(s.elapsed_time(e))
        del kept
        times = sorted(times[1:])
        return times[len(times) // 2]

    return replayed_ms(dots), replayed_ms(builds), len(dots), len(builds)


def run(model_name="opt-1.3b", seq_len=512, batch=1, iters=5, warmup=2, decimal_places=2, compress_threshold=0.5,
        seed=123, dense=True, graph=True, fuse_qkv=False, quantize_lm_head=False):
    from bsipytorch_amd import bsi_ops, linear

    assert torch.cuda.is_available(), "needs the GPU"
    layers, hidden, heads, ffn, vocab = SHAPES[model_name]
    model = build_model(model_name, seed, "cuda")
    g = torch.Generator().manual_seed(seed)
    input_ids = torch.randint(0, vocab, (batch, seq_len), generator=g).cuda()
    tokens = batch * seq_len
    res = {"model": model_name, "layers": layers, "hidden": hidden, "heads": heads, "ffn": ffn, "vocab": vocab,
           "batch": batch, "seq_len": seq_len, "decimal_places": decimal_places,
           "compress_threshold": compress_threshold}

    if dense:
        med, best = time_forward(model, input_ids, iters, warmup)
        res["dense_fp32_fwd_ms"] = med
        res["dense_fp32_tokens_per_s"] = tokens / (med * 1e-3)

    t0 = time.perf_counter()
    linear.quantize_model_bsi(model, decimalPlaces=decimal_places, compress_threshold=compress_threshold, verbose=False,
                              fuse_qkv=fuse_qkv, skip_lm_head=not quantize_lm_head)
    res["fuse_qkv"] = bool(fuse_qkv)
    res["lm_head"] = "bsi" if quantize_lm_head else "dense"
    torch.cuda.synchronize()
    res["key_build_s"] = time.perf_counter() - t0
    summary = linear.summarize_bsi_model(model)
    res["num_bsi_layers"] = summary["num_quantized_layers"]
    res["bsi_key_bytes"] = summary["total_bsi_bytes"]
    res["dense_linear_bytes"] = summary["total_dense_bytes"]

    # pass 1: no per-call events -> tokens/s
    os.environ["BSI_PROFILE"] = "0"
    bsi_ops._reset_flag_cache()
    med, best = time_forward(model, input_ids, iters, warmup)
    res["bsi_fwd_ms"] = med
    res["bsi_fwd_ms_min"] = best
    res["bsi_tokens_per_s"] = tokens / (med * 1e-3)

    # pass 1b: the same forward captured once into a HIP graph and replayed (no host work per layer).
    # Replays are checked against the eager logits, with eager work in between, as graph replays must be.
    if graph and bsi_ops._flags()["bits_q"] == 0:
        res["bsi_graph_fwd_ms"] = None  # decimal-mode builds read a scalar back from the device: not recordable
    elif graph:
        with torch.no_grad():
            eager = model(input_ids).clone()
            graphed = linear.GraphedForward(model, input_ids)
            same = True
            times = []
            for _ in range(max(iters, 3)):
                s_evt, e_evt = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                s_evt.record()
                static_out = graphed(graphed.static_inputs[0])  # the recorded input: the replay alone is timed
                e_evt.record()
                torch.cuda.synchronize()
                times.append(s_evt.elapsed_time(e_evt))
                same = same and bool(torch.equal(static_out, eager))
                same = same and bool(torch.equal(model(input_ids), eager))  # eager work between replays
            times.sort()
            res["bsi_graph_fwd_ms"] = times[len(times) // 2]
            res["bsi_graph_tokens_per_s"] = tokens / (times[len(times) // 2] * 1e-3)
            res["graph_replays_match_eager"] = same

    # pass 2a: GPU time of the dots and of the query builds by themselves, unsynchronised -> the shares of the forward
    if graph and bsi_ops._flags()["bits_q"] != 0 and res.get("bsi_graph_fwd_ms"):
        dot_gpu_ms, build_gpu_ms, n_dots, n_builds = kernel_time_of_dots_and_builds(model, input_ids)
        res["dot_gpu_ms_per_prefill"] = dot_gpu_ms
        res["query_build_gpu_ms_per_prefill"] = build_gpu_ms
        res["dot_launches_per_prefill"], res["query_builds_per_prefill"] = n_dots, n_builds
        res["dot_share_of_graph_fwd"] = dot_gpu_ms / res["bsi_graph_fwd_ms"]
        res["query_build_share_of_graph_fwd"] = build_gpu_ms / res["bsi_graph_fwd_ms"]

    # pass 2: per-call device events on the dot and the builder (each call synchronised, so launch latency is in)
    os.environ["BSI_PROFILE"] = "1"
    bsi_ops._reset_flag_cache()
    time_forward(model, input_ids, 1, 1)
    linear.reset_bsi_dot_counters(model)
    prof_med, _ = time_forward(model, input_ids, iters, 0)
    dot_ms = linear.sum_bsi_dot_counters(model) / 1e6 / iters
    build_kernel_ms = linear.sum_bsi_build_kernel_counters(model) / 1e6 / iters
    build_host_ms = linear.sum_bsi_build_counters(model) / 1e6 / iters
    os.environ["BSI_PROFILE"] = "0"
    bsi_ops._reset_flag_cache()
    res["profiled_fwd_ms"] = prof_med
    res["dot_ms_per_prefill"] = dot_ms
    res["query_build_kernel_ms_per_prefill"] = build_kernel_ms
    res["query_build_host_ms_per_prefill"] = build_host_ms
    res["dot_share_of_fwd"] = dot_ms / med
    res["query_build_share_of_fwd"] = build_kernel_ms / med
    bitmacs = 42.0 * tokens * layers * (4 * hidden * hidden + 2 * hidden * ffn)
    res["dot_effective_bitop_TOPS"] = 2.0 * bitmacs / (dot_ms * 1e-3) / 1e12 if dot_ms > 0 else None
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", default="opt-1.3b", choices=sorted(SHAPES))
    ap.add_argument("--seq_len", type=int, default=512)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--iters", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--decimal_places", type=int, default=2)
    ap.add_argument("--compress_threshold", type=float, default=0.5)
    ap.add_argument("--seed", type=int, default=123)
    ap.add_argument("--no_dense", action="store_true")
    ap.add_argument("--no_graph", action="store_true", help="skip the HIP-graph replay leg")
    ap.add_argument("--fuse_qkv", action="store_true", help="one dot for q_proj, k_proj and v_proj of a layer")
    ap.add_argument("--quantize_lm_head", action="store_true",
                    help="also replace lm_head (the reference's harness keeps it dense; this is an extra figure)")
    a = ap.parse_args()
    print(json.dumps(run(a.model, a.seq_len, a.batch, a.iters, a.warmup, a.decimal_places, a.compress_threshold,
                         a.seed, not a.no_dense, not a.no_graph, a.fuse_qkv, a.quantize_lm_head)))


if __name__ == "__main__":
    main()
