"""Host-side contracts of the BSI-linear drop-in that need the GPU: workspaces whose addresses a recorded HIP
graph holds stay valid when later calls need larger ones, and the layer works on tensors that carry no version
counter (``torch.inference_mode()``), as the reference layer does (verify_accuracy_bsi.py:118-215)."""
import os

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


def _capture(fn, warm):
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        warm()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = fn()
    return g, out


def test_graph_replay_survives_a_larger_eager_call(ops):
    """Capture a forward at 64 rows, then run an eager forward that needs a workspace sixteen times larger, then
    replay: the replay must still build into memory it owns and give the eager bits."""
    from bsipytorch_amd import linear

    torch.manual_seed(3)
    model = torch.nn.ModuleList([torch.nn.Linear(1024, 320).cuda(), torch.nn.Linear(1024, 192).cuda()])
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    ops._linear_ws.clear()
    ops._reserved_linear_shapes.clear()
    x = torch.randn(64, 1024, device="cuda")
    big = torch.randn(4096, 1024, device="cuda")
    with torch.no_grad():
        want = [m(x).clone() for m in model]
        static_x = x.clone()
        linear.forget_shared_builds()
        g, outs = _capture(lambda: [m(static_x) for m in model], lambda: [m(static_x) for m in model])
        linear.forget_shared_builds()
        small_bytes = ops._linear_ws[x.device.index]["bytes"]
        captured_ptr = ops._linear_ws[x.device.index]["capture_buf"].data_ptr()
        big_out = [m(big) for m in model]                     # grows both workspaces
        assert ops._linear_ws[x.device.index]["bytes"] > small_bytes
        assert any(t.data_ptr() == captured_ptr for t in ops._retired_workspaces)
        # memory the allocator hands out now must not be what the recorded launches write
        fill = [torch.full((small_bytes,), 0x5A, dtype=torch.uint8, device="cuda") for _ in range(4)]
        for rep in range(3):
            static_x.copy_(x * (rep + 1))
            g.replay()
            torch.cuda.synchronize()
            assert all(torch.equal(a, m(x * (rep + 1))) for a, m in zip(outs, model))
            assert all(bool((t == 0x5A).all()) for t in fill)
        static_x.copy_(x)
        g.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(outs, want))
        assert all(torch.equal(a, m(big)) for a, m in zip(big_out, model))


def test_dot_workspace_is_retired_not_freed_after_a_capture(ops):
    """The dot's own scratch buffer (decimal digit products): a buffer a capture has used is kept when a larger one
    replaces it, and growing inside a capture raises."""
    dev = torch.device("cuda", torch.cuda.current_device())
    ops._workspace.clear()
    a = ops._get_workspace(1 << 16, dev)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        inside = ops._get_workspace(1 << 12, dev)
        inside[:16].zero_()
    assert inside.data_ptr() == a.data_ptr() and ops._workspace[dev]["captured"]
    before = len(ops._retired_workspaces)
    b = ops._get_workspace(1 << 20, dev)
    assert b.data_ptr() != a.data_ptr() and len(ops._retired_workspaces) == before + 1
    assert ops._retired_workspaces[-1].data_ptr() == a.data_ptr()
    g2 = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="larger workspace"):
        with torch.cuda.graph(g2):
            ops._get_workspace(1 << 24, dev)
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("rows", [3, 48])
def test_layer_and_fused_qkv_under_inference_mode(ops, monkeypatch, dtype, rows):
    """Inference tensors keep no version counter: nothing may read it, builds are not shared, results are the bits of
    the same forward under no_grad (few-rows kernel, one-call path and the two-call path)."""
    from bsipytorch_amd import linear

    class Attn(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj = torch.nn.Linear(512, 128)
            self.k_proj = torch.nn.Linear(512, 128)
            self.v_proj = torch.nn.Linear(512, 192, bias=False)
            self.out_proj = torch.nn.Linear(512, 100)

        def forward(self, x):
            return self.q_proj(x), self.k_proj(x), self.v_proj(x), self.out_proj(x)

    torch.manual_seed(9)
    plain = Attn().cuda()
    fused = Attn().cuda()
    fused.load_state_dict(plain.state_dict())
    linear.quantize_model_bsi(plain, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    linear.quantize_model_bsi(fused, decimalPlaces=2, compress_threshold=0.5, verbose=False, fuse_qkv=True)
    x = torch.randn(rows, 512, device="cuda").to(dtype)
    for one_call in ("1", "0"):
        monkeypatch.setenv("BSI_LINEAR_ONE_CALL", one_call)
        linear.forget_shared_builds()
        with torch.no_grad():
            want = [t.clone() for t in plain(x)]
        linear.forget_shared_builds()
        with torch.no_grad():
            want2 = [t.clone() for t in plain(x + 1.0)]
        linear.forget_shared_builds()
        with torch.inference_mode():
            for model in (plain, fused):
                xi = x.clone()                  # an inference tensor
                assert xi.is_inference()
                got = model(xi)
                assert all(torch.equal(a, b) for a, b in zip(got, want))
                xi.add_(1.0)                    # in-place work on it must not be mistaken for "unchanged"
                got2 = model(xi)
                assert all(torch.equal(a, b) for a, b in zip(got2, want2))


@pytest.mark.parametrize("rows", [2, 40])
@pytest.mark.parametrize("fuse", [False, True])
def test_layer_with_its_bias_on_the_host(ops, rows, fuse):
    """A layer quantised while it lives on the CPU keeps its bias there (the reference moves it per call,
    verify_accuracy_bsi.py:207-211).  No kernel may be handed that host pointer: the few-rows kernel, the one-call path
    and the fused q/k/v group add such a bias afterwards, with the result of a layer whose bias is on the device; the
    library-level entry points refuse it."""
    import torch.nn as nn
    from bsipytorch_amd.linear import BSIQuantizedLinear, forget_shared_builds, fuse_sibling_layers

    torch.manual_seed(5)
    D, R = 512, (128 if fuse else 100)  # siblings are stacked only when their key counts are multiples of 64

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj, self.k_proj, self.v_proj = nn.Linear(D, R), nn.Linear(D, R), nn.Linear(D, R)

    def quantised(move_bias):
        torch.manual_seed(6)
        blk = Block()
        for name in ("q_proj", "k_proj", "v_proj"):
            layer = BSIQuantizedLinear(getattr(blk, name), decimalPlaces=2, compress_threshold=0.5)
            if move_bias:
                layer.cuda()  # moves the bias buffer; the keys are on the device either way
            setattr(blk, name, layer)
        if fuse:
            assert fuse_sibling_layers(blk) == 1
        return blk

    x = torch.randn(rows, D, device="cuda")
    host, dev = quantised(False), quantised(True)
    assert not host.q_proj.bias.is_cuda and dev.q_proj.bias.is_cuda
    for name in ("q_proj", "k_proj", "v_proj"):
        a, b = getattr(host, name)(x), getattr(dev, name)(x)
        torch.cuda.synchronize()
        assert torch.equal(a, b), name
    forget_shared_builds()
    keys = dev.q_proj._bsi_keys_cuda
    with pytest.raises(RuntimeError, match="bias must be"):
        ops.linear_cuda(x, keys, 2, bias=host.q_proj.bias.detach())
    if rows <= ops.FUSED_LINEAR_MAX_ROWS:
        with pytest.raises(RuntimeError, match="bias must be"):
            ops.linear_few_rows_cuda(x, keys, 2, bias=host.q_proj.bias.detach())
    with pytest.raises(RuntimeError, match="bias must be"):
        ops.linear_cuda(x, keys, 2, bias=torch.zeros(R + 1, device="cuda"))
    forget_shared_builds()


@pytest.mark.parametrize("rows", [2, 96])
def test_graphed_forward_replays_match_eager(ops, rows):
    """linear.GraphedForward: a small model of BSI layers recorded once; every replay, on fresh inputs and with eager
    forwards of the same model in between, gives the eager bits; a call with another shape is refused."""
    from bsipytorch_amd import linear

    torch.manual_seed(rows)
    model = torch.nn.Sequential(torch.nn.Linear(512, 1024), torch.nn.ReLU(), torch.nn.Linear(1024, 256)).cuda()
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    xs = [torch.randn(rows, 512, device="cuda") * (i + 1) for i in range(4)]
    with torch.no_grad():
        want = [model(x).clone() for x in xs]
        graphed = linear.GraphedForward(model, xs[0])
        for rep in range(2):
            for x, w in zip(xs, want):
                got = graphed(x)
                torch.cuda.synchronize()
                assert torch.equal(got, w)
                assert torch.equal(model(xs[(rep + 1) % 4]), want[(rep + 1) % 4])  # eager work between replays
        with pytest.raises(ValueError):
            graphed(torch.randn(rows + 1, 512, device="cuda"))
        with pytest.raises(ValueError):
            graphed(xs[0], xs[1])


def test_eager_forwards_on_two_streams_build_into_their_own_workspaces(ops):
    """Two streams run forwards of two layers at the same time: each stream's query build goes into a workspace of its
    own (one shared buffer would let one stream's build overwrite the operands the other stream's dot is about to
    read), and every output has the bits of the same forward run alone."""
    from bsipytorch_amd import linear

    torch.manual_seed(12)
    layers = [torch.nn.Linear(1024, 768).cuda(), torch.nn.Linear(1024, 512).cuda()]
    model = torch.nn.ModuleList(layers)
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    ops._linear_ws.clear()
    xs = [torch.randn(256, 1024, device="cuda") * (i + 1) for i in range(6)]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    with torch.no_grad():
        want = [[model[j](x).clone() for x in xs] for j in range(2)]
        torch.cuda.synchronize()
        got = [[None] * len(xs) for _ in range(2)]
        for rep in range(3):
            for i, x in enumerate(xs):
                for j, s in enumerate(streams):
                    s.wait_stream(torch.cuda.current_stream())
                    with torch.cuda.stream(s):
                        got[j][i] = model[j](x)
            torch.cuda.synchronize()
            for j in range(2):
                for i in range(len(xs)):
                    assert torch.equal(got[j][i], want[j][i]), (rep, j, i)
    eager = ops._linear_ws[xs[0].device.index]["eager"]
    handles = {s.cuda_stream for s in streams}
    assert handles <= set(eager), (handles, set(eager))
    assert len({eager[h][0].data_ptr() for h in handles}) == 2


def test_graphed_forward_refuses_what_cannot_be_recorded(ops, monkeypatch):
    """Decimal-mode builds read a scalar back from the device and BSI_PROFILE=1 synchronises: GraphedForward says so
    up front instead of failing inside the capture."""
    from bsipytorch_amd import linear

    model = torch.nn.Sequential(torch.nn.Linear(256, 64)).cuda()
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False)
    x = torch.randn(8, 256, device="cuda")
    for name, value, text in (("BSI_FIXED_BITS", "0", "decimal-mode"), ("BSI_PROFILE", "1", "BSI_PROFILE")):
        monkeypatch.setenv(name, value)
        ops._reset_flag_cache()
        with pytest.raises(RuntimeError, match=text):
            linear.GraphedForward(model, x)
        monkeypatch.delenv(name)
        ops._reset_flag_cache()
    with torch.no_grad():
        assert torch.equal(linear.GraphedForward(model, x)(x), model(x))


@pytest.mark.parametrize("fuse", [False, True])
def test_a_second_capture_on_the_same_static_input_builds_anew(ops, fuse):
    """Two graphs recorded by hand, one after the other, with no forget_shared_builds() in between, the second starting
    on the tensor the first ended on (same address, shape and version): the second graph carries its own query build,
    so its replays follow what is copied into the static input."""
    from bsipytorch_amd import linear

    torch.manual_seed(17)
    model = torch.nn.ModuleDict({n: torch.nn.Linear(512, 128).cuda() for n in ("q_proj", "k_proj", "v_proj")})
    linear.quantize_model_bsi(model, decimalPlaces=2, compress_threshold=0.5, verbose=False, fuse_qkv=fuse)
    x0, x1 = torch.randn(96, 512, device="cuda"), torch.randn(96, 512, device="cuda")
    with torch.no_grad():
        want0 = [model[n](x0).clone() for n in ("q_proj", "k_proj", "v_proj")]
        want1 = [model[n](x1).clone() for n in ("q_proj", "k_proj", "v_proj")]
        static_x = x0.clone()
        fwd = lambda: [model[n](static_x) for n in ("q_proj", "k_proj", "v_proj")]  # noqa: E731
        g1, out1 = _capture(fwd, fwd)
        g2, out2 = _capture(fwd, lambda: None)   # nothing in between: same storage, same version counter
        static_x.copy_(x1)
        g2.replay()
        torch.cuda.synchronize()
        for got, want in zip(out2, want1):
            assert torch.equal(got, want)
        static_x.copy_(x0)
        g1.replay()
        g2.replay()
        torch.cuda.synchronize()
        for a, b, want in zip(out1, out2, want0):
            assert torch.equal(a, want) and torch.equal(b, want)
    linear.forget_shared_builds()
