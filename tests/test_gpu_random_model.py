"""A seeded sweep of a small transformer-shaped block (q/k/v/out projections, fc1, fc2, a dense head) through
quantize_model_bsi in every way a model is used: eager, with fresh query builds, under inference_mode, recorded into a
HIP graph and replayed with eager work in between, saved and loaded again.  All of them must give the same bits, and
those bits must be the dense model's output up to the quantisation error."""
import copy
import os
import numpy as np
import pytest
import torch
import torch.nn as nn

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


class Block(nn.Module):
    def __init__(self, hidden, ffn, bias):
        super().__init__()
        self.q_proj = nn.Linear(hidden, hidden, bias=bias)
        self.k_proj = nn.Linear(hidden, hidden, bias=bias)
        self.v_proj = nn.Linear(hidden, hidden, bias=bias)
        self.out_proj = nn.Linear(hidden, hidden, bias=bias)
        self.fc1 = nn.Linear(hidden, ffn, bias=bias)
        self.fc2 = nn.Linear(ffn, hidden, bias=bias)
        self.lm_head = nn.Linear(hidden, 50, bias=False)

    def forward(self, x):
        a = torch.tanh(self.q_proj(x)) * torch.sigmoid(self.k_proj(x)) + self.v_proj(x)
        x = x + self.out_proj(a)
        x = x + self.fc2(torch.relu(self.fc1(x)))
        return self.lm_head(x)


@pytest.mark.parametrize("seed", range(24))
def test_block_modes_agree(ops, seed, tmp_path):
    from bsipytorch_amd.linear import GraphedForward, quantize_model_bsi, forget_shared_builds, save_bsi_model, load_bsi_model
    rng = np.random.default_rng(300 + seed)
    hidden = int(rng.choice([64, 128, 192, 256, 320, 512]))
    ffn = int(rng.choice([256, 512, 768, 1024]))
    rows = int(rng.choice([1, 2, 4, 5, 16, 40, 130]))
    dt = [torch.float32, torch.float16, torch.bfloat16][int(rng.integers(0, 3))]
    bias = bool(rng.integers(0, 2))
    fuse = bool(rng.integers(0, 2))
    on_gpu_first = bool(rng.integers(0, 2))
    three_d = bool(rng.integers(0, 2))
    torch.manual_seed(seed)
    dense = Block(hidden, ffn, bias).to(dt)
    with torch.no_grad():
        for p in dense.parameters():
            p.mul_(0.5)
    base = copy.deepcopy(dense)
    if on_gpu_first:
        dense = dense.cuda()
    model = quantize_model_bsi(dense, 2, compress_threshold=0.5, verbose=False, fuse_qkv=fuse).cuda()
    x = torch.randn((2, rows, hidden) if three_d else (rows, hidden), device="cuda").to(dt)
    with torch.no_grad():
        y0 = model(x).clone()
        forget_shared_builds()
        y1 = model(x.clone()).clone()
    assert torch.equal(y0, y1)
    assert torch.isfinite(y0.float()).all()
    with torch.inference_mode():
        y2 = model(x.clone()).clone()
    assert torch.equal(y0, y2)
    # against the dense model: the quantisation error only
    with torch.no_grad():
        yd = base.cuda()(x).float()
    rel = float((y0.float() - yd).norm() / (yd.norm() + 1e-6))
    assert rel < 0.6, rel
    # recorded into a graph and replayed, eager work between the replays
    graphed = GraphedForward(model, x)
    for _ in range(3):
        yg = graphed(x)
        torch.cuda.synchronize()
        assert torch.equal(yg, y0)
        with torch.no_grad():
            model(torch.randn_like(x))
    # save and load
    d = str(tmp_path / "m")
    save_bsi_model(model, d)
    fresh = load_bsi_model(copy.deepcopy(base), d).cuda()
    with torch.no_grad():
        y3 = fresh(x.clone())
    assert torch.equal(y0, y3)
    forget_shared_builds()
