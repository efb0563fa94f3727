"""The HIP path at the full sizes of the benchmark configurations, against the CPU oracle IN FULL (every output
element: with all host threads the oracle needs 0.2 s for the FC1-like shape and 1.5 s for the largest one), with
the tile the launcher picks by itself:

  * FC1-like Q512 x R8192 x D2048 with outlier columns, FC2-like Q512 x R2048 x D8192 with ReLU queries: whole
    fp32 output bit-identical to the oracle, both cores identical, integer accumulators of sampled chunks against an
    independent fp64 matrix product, and size-independent properties (row permutations of either operand, a common
    power-of-two factor on the chunk scales, a chunk switched off by a zero scale or by empty planes);
  * OPT-1.3B projection 512 x 2048 x 2048 and a two-layer OPT-1.3B-shaped decoder (hidden 2048, 32 heads, FFN 8192)
    with every linear layer replaced: each layer's output against oracle dot + bias on that layer's own input;
  * OPT-6.7B layer shapes 4096 x 4096, 16384 x 4096, 4096 x 16384 at 1, 16, 128 and 512 query rows.

The stated tolerance for fp32 outputs is 1e-5 relative; the asserts ask for identical bits, which implies it.
"""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

FP32_RTOL = 1e-5


@pytest.fixture()
def ops(monkeypatch):
    from bsipytorch_amd import bsi_ops

    for k in list(os.environ):
        if k.startswith("BSI_"):
            monkeypatch.delenv(k)
    bsi_ops._reset_flag_cache()
    yield bsi_ops
    bsi_ops._reset_flag_cache()


def _oracle_out(oracle, X: np.ndarray, kb) -> np.ndarray:
    qb = oracle.build_queries(X)
    _, want = oracle.dot_fixed(qb["words"], qb["scales"], kb["words"], kb["scales"], oracle.scale_inv(2, 2), want_ints=False)
    return want


def _scales_of(qcap):
    if qcap.chunk_scales is not None and qcap.chunk_scales.numel() > 0:
        return qcap.chunk_scales, int(qcap.chunk_scales.shape[1])
    return qcap.row_scales, 1


def _valu_out(ops, qcap, kcap):
    from bsipytorch_amd import _lib

    sc, stride = _scales_of(qcap)
    out, _ = ops._dot(qcap.words, qcap.ints8, sc, stride, qcap.Sa, qcap.W, kcap, qcap.Q, qcap.decimals, core=_lib.CORE_VALU)
    return out


def _fp64_chunk_ints(qcap, kcap, K, chunk_ids):
    """Integer dots of the quantised values of the given chunks in fp64 on the GPU (exact: every partial sum is far
    below 2^53); the query values are read back from the int8 operand, the key values re-derived from the floats
    with torch arithmetic that shares nothing with the library or the oracle."""
    D = K.shape[1]
    e = torch.arange(D, device="cuda")
    pos = (e // 32) * 32 + ((e % 32) % 8) * 4 + (e % 32) // 8
    a = qcap.ints8[:, pos].to(torch.float64) / 2.0
    kx = K.cuda().double() * 100.0
    rk = torch.sign(kx) * torch.floor(kx.abs() + 0.5)
    sh = kcap.shifts.to(torch.float64).unsqueeze(1)
    b = torch.sign(rk) * torch.floor((rk.abs() + torch.where(sh > 0, 2.0 ** (sh - 1), torch.zeros_like(sh))) / 2.0 ** sh)
    b = b.clamp(-32, 31)
    return {c: a[:, c * 256:(c + 1) * 256] @ b[:, c * 256:(c + 1) * 256].T for c in chunk_ids}


def _clone_queries(ops, qcap, **changes):
    h = ops.PrebuiltBSIQueryBatchCUDA()
    h.__dict__.update(qcap.__dict__)
    h.__dict__.update(changes)
    return h


@pytest.mark.parametrize("name,Q,R,D,kind,chunks_checked", [("fc1", 512, 8192, 2048, "outliers", (0, 3, 7)),
                                                            ("fc2", 512, 2048, 8192, "relu", (0, 13, 31))])
def test_headline_shapes_in_full_against_the_oracle(ops, oracle, name, Q, R, D, kind, chunks_checked):
    torch.manual_seed(123)
    X = torch.randn(Q, D)
    if kind == "outliers":
        X[:, torch.randperm(D)[:2]] *= 20.0
    else:
        X = torch.relu(X)
    K = torch.randn(R, D) * 0.02
    K[5] *= 40.0                                              # one key row with its own scale
    kcap, *_ = ops.build_bsi_keys_cuda(K, 2, 0.5)
    qcap = ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.5)
    out = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)[0]
    kb = oracle.build_keys(K.numpy())
    want = _oracle_out(oracle, X.numpy(), kb)
    got = out.cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=FP32_RTOL, atol=0)
    np.testing.assert_array_equal(got, want)                  # the whole fp32 chain, every element
    assert torch.equal(_valu_out(ops, qcap, kcap), out)       # popcount core: the same bits
    ints, out_dump = ops.debug_chunk_ints(qcap, kcap, "mfma")
    assert torch.equal(out_dump, out)
    for c, exact in _fp64_chunk_ints(qcap, kcap, K, chunks_checked).items():
        assert torch.equal(ints[:, :, c].to(torch.float64), exact)
    del ints
    # permuting query rows permutes output rows; permuting key rows permutes output columns
    qp = torch.randperm(Q)
    qcap_p = ops.build_bsi_queries_cuda_batch_packed(X[qp].cuda(), 2, 0.5)
    assert torch.equal(ops.batch_dot_product_multiquery_cuda_batch_caps(qcap_p, kcap)[0], out[qp.cuda()])
    kp = torch.randperm(R)
    kcap_p, *_ = ops.build_bsi_keys_cuda(K[kp], 2, 0.5)
    assert torch.equal(ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap_p)[0], out[:, kp.cuda()])
    # a common power-of-two factor on every chunk scale comes out as that factor, exactly
    scaled = _clone_queries(ops, qcap, chunk_scales=qcap.chunk_scales * 8.0)
    assert torch.equal(ops.batch_dot_product_multiquery_cuda_batch_caps(scaled, kcap)[0], out * 8.0)
    # a chunk switched off by a zero scale gives what the same chunk with empty planes gives
    c = chunks_checked[1]
    sc0 = qcap.chunk_scales.clone()
    sc0[:, c] = 0.0
    off_by_scale = ops.batch_dot_product_multiquery_cuda_batch_caps(_clone_queries(ops, qcap, chunk_scales=sc0), kcap)[0]
    words0, ints0 = qcap.words.clone(), qcap.ints8.clone()
    words0[:, :, 4 * c:4 * c + 4] = 0
    ints0[:, 256 * c:256 * c + 256] = 0
    off_by_planes = ops.batch_dot_product_multiquery_cuda_batch_caps(_clone_queries(ops, qcap, words=words0, ints8=ints0), kcap)[0]
    assert torch.equal(off_by_scale, off_by_planes) and not torch.equal(off_by_scale, out)
    Xz = X.clone()
    Xz[:, 256 * c:256 * c + 256] = 0.0
    np.testing.assert_array_equal(off_by_planes.cpu().numpy(), _oracle_out(oracle, Xz.numpy(), kb))


def test_opt13b_projection_shape_in_full(ops, oracle):
    """512 tokens through a 2048 -> 2048 projection (q/k/v/out of OPT-1.3B), with bias in the dot's epilogue."""
    torch.manual_seed(11)
    Q, R, D = 512, 2048, 2048
    X, K, bias = torch.randn(Q, D), torch.randn(R, D) * 0.02, torch.randn(R)
    kcap, *_ = ops.build_bsi_keys_cuda(K, 2, 0.5)
    qcap = ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.5)
    out = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)[0]
    want = _oracle_out(oracle, X.numpy(), oracle.build_keys(K.numpy()))
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    assert torch.equal(_valu_out(ops, qcap, kcap), out)
    with_bias = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap, bias.cuda())[0]
    np.testing.assert_array_equal(with_bias.cpu().numpy(), want + bias.numpy()[None, :])
    assert torch.equal(ops.linear_cuda(X.cuda(), kcap, 2, bias.cuda()), with_bias)


@pytest.mark.parametrize("fuse_qkv", [False, True])
def test_opt13b_shaped_two_layer_decoder_layer_by_layer(ops, oracle, fuse_qkv):
    """Two decoder layers of the OPT-1.3B architecture (hidden 2048, 32 heads, FFN 8192) built from a local
    OPTConfig with random weights and non-zero biases, every linear layer replaced by the BSI drop-in, one prefill
    of 512 tokens: each BSI layer's output must be the oracle's dot of that layer's own input with that layer's
    keys, plus its bias -- bit for bit, all twelve layers (four 2048 x 2048 projections, fc1 and fc2 per block)."""
    from transformers import OPTConfig, OPTModel

    from bsipytorch_amd import linear

    torch.manual_seed(2)
    cfg = OPTConfig(vocab_size=4096, hidden_size=2048, num_hidden_layers=2, ffn_dim=8192, num_attention_heads=32,
                    max_position_embeddings=512, word_embed_proj_dim=2048, do_layer_norm_before=True)
    model = OPTModel(cfg).eval()
    with torch.no_grad():
        for n, p in model.named_parameters():
            if "layer_norm" in n:
                continue
            p.normal_(0.0, 0.02)                              # weights and biases alike
    model = model.cuda()
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False, fuse_qkv=fuse_qkv)
    layers = {n: m for n, m in model.named_modules() if isinstance(m, linear.BSIQuantizedLinear)}
    assert len(layers) == 12
    seen = {}
    hooks = [m.register_forward_hook(lambda mod, args, out, n=n: seen.__setitem__(n, (args[0].detach().clone(), out.detach().clone())))
             for n, m in layers.items()]
    ids = torch.randint(0, 4096, (1, 512), device="cuda")
    with torch.no_grad():
        hidden = model(ids).last_hidden_state
    for h in hooks:
        h.remove()
    assert torch.isfinite(hidden).all() and len(seen) == 12
    for n, m in layers.items():
        x, y = seen[n]
        x2 = x.reshape(-1, x.shape[-1]).float().cpu().numpy()
        kb = oracle.build_keys(m.weight_fp32.numpy())
        want = _oracle_out(oracle, x2, kb) + m.bias_fp32.numpy()[None, :]
        np.testing.assert_array_equal(y.reshape(-1, y.shape[-1]).cpu().numpy(), want, err_msg=n)


def test_opt13b_shaped_full_stack(ops, oracle):
    """The whole C4 configuration as the benchmark builds it (24 decoder layers, hidden 2048, 32 heads, FFN 8192,
    vocab 50272, 144 BSI layers, one prefill of 512 tokens): the layers sampled from the first, a middle and the last
    block equal the oracle's dot of their own input plus their bias bit for bit, the logits are finite, and the
    forward replayed from a HIP graph gives the eager logits."""
    from bsipytorch_amd import linear
    from bsipytorch_amd.benchmarks import benchmark_opt_prefill as bench_model

    model = bench_model.build_model("opt-1.3b", 123, "cuda")
    with torch.no_grad():
        for n, p in model.named_parameters():
            if n.endswith("bias") and "layer_norm" not in n:
                p.normal_(0.0, 0.02, generator=torch.Generator(device="cuda").manual_seed(len(n)))
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    layers = {n: m for n, m in model.named_modules() if isinstance(m, linear.BSIQuantizedLinear)}
    assert len(layers) == 144
    sampled = ["layers.0.self_attn.q_proj", "layers.0.fc2", "layers.11.self_attn.out_proj", "layers.11.fc1",
               "layers.23.self_attn.v_proj", "layers.23.fc2"]
    seen = {}
    hooks = [layers[n].register_forward_hook(
        lambda mod, args, out, n=n: seen.__setitem__(n, (args[0].detach().clone(), out.detach().clone()))) for n in sampled]
    ids = torch.randint(0, 50272, (1, 512), generator=torch.Generator().manual_seed(123)).cuda()
    with torch.no_grad():
        logits = model(ids).clone()
    for h in hooks:
        h.remove()
    assert logits.shape == (1, 512, 50272) and torch.isfinite(logits).all()
    for n in sampled:
        x, y = seen[n]
        m = layers[n]
        kb = oracle.build_keys(m.weight_fp32.numpy())
        want = _oracle_out(oracle, x.reshape(-1, x.shape[-1]).float().cpu().numpy(), kb) + m.bias_fp32.numpy()[None, :]
        np.testing.assert_array_equal(y.reshape(-1, y.shape[-1]).cpu().numpy(), want, err_msg=n)
    with torch.no_grad():
        graphed = linear.GraphedForward(model, ids)
        for _ in range(2):
            assert torch.equal(graphed(ids), logits)
            assert torch.equal(model(ids), logits)   # eager work between the replays
    del graphed, model
    torch.cuda.empty_cache()


_C5_SHAPES = {"attn": (4096, 4096), "fc1": (16384, 4096), "fc2": (4096, 16384)}
_c5_cache = {}


def _c5_keys(ops, oracle, name):
    """Keys of one OPT-6.7B layer shape, built once per test session (floats, oracle planes, device keyset)."""
    if name not in _c5_cache:
        _c5_cache.clear()                                     # one shape at a time: the floats alone are 256 MiB
        R, D = _C5_SHAPES[name]
        g = torch.Generator().manual_seed(R + D)
        K = torch.randn(R, D, generator=g) * 0.02
        K[R // 3] *= 30.0
        kcap, *_ = ops.build_bsi_keys_cuda(K, 2, 0.5)
        _c5_cache[name] = (K, oracle.build_keys(K.numpy()), kcap)
    return _c5_cache[name]


@pytest.mark.parametrize("Q", [1, 16, 128, 512])
@pytest.mark.parametrize("name", ["attn", "fc1", "fc2"])
def test_opt67b_layer_shapes_in_full(ops, oracle, name, Q):
    R, D = _C5_SHAPES[name]
    K, kb, kcap = _c5_keys(ops, oracle, name)
    g = torch.Generator().manual_seed(Q * 7 + D)
    X = torch.randn(Q, D, generator=g)
    qcap = ops.build_bsi_queries_cuda_batch_packed(X.cuda(), 2, 0.5)
    out = ops.batch_dot_product_multiquery_cuda_batch_caps(qcap, kcap)[0]
    want = _oracle_out(oracle, X.numpy(), kb)
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=FP32_RTOL, atol=0)
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    if Q >= 128:
        assert torch.equal(_valu_out(ops, qcap, kcap), out)
    if Q == 128:
        ints, _ = ops.debug_chunk_ints(qcap, kcap, "mfma")
        for c, exact in _fp64_chunk_ints(qcap, kcap, K, (0, D // 256 - 1)).items():
            assert torch.equal(ints[:, :, c].to(torch.float64), exact)


def test_c5_cache_released():
    _c5_cache.clear()
