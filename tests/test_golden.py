"""The committed c1 fixture: the oracle reproduces it on CPU, the HIP path reproduces it on the GPU."""
import hashlib
import json
import os

import pytest
import torch

import oracle
from _inputs import CONFIGS, make_inputs

FIX = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "c1_seed0.json")))


def _digest(t):
    return hashlib.sha256(t.detach().contiguous().numpy().tobytes()).hexdigest()[:16]


def test_inputs_are_the_ones_the_fixture_was_made_from():
    """The expected rows mean something only for the inputs they were computed from: the seeded draw must still give
    the tensors whose digests the fixture records."""
    t = make_inputs(CONFIGS["c1"], seed=0)
    assert {k: _digest(v) for k, v in t.items()} == FIX["inputs_sha256_16"]


def _check(y, dx, dp, dw1, dw2, routing, tol):
    rows = FIX["rows"]
    if routing is not None:
        for name, t in zip(("sorted_expert_idxs", "sorted_scattered_idxs", "expert_offsets"), routing):
            assert t.cpu().tolist() == FIX["routing"][name]                       # bit-exact
    assert torch.allclose(y.cpu()[rows, :8], torch.tensor(FIX["Y_rows"]), atol=tol)
    assert torch.allclose(dx.cpu()[rows, :8], torch.tensor(FIX["dX_rows"]), atol=tol)
    assert torch.allclose(dp.cpu()[rows], torch.tensor(FIX["dg_rows"]), atol=tol)
    for name, t in (("Y", y), ("dX", dx), ("dg", dp), ("dW1", dw1), ("dW2", dw2)):
        assert abs(float(t.double().sum()) - FIX["sums"][name]) < tol * 100 * max(1.0, abs(FIX["sums"][name]))
    assert abs(float(dw1.double().abs().sum()) - FIX["sums"]["dW1_abs"]) < 1e-3 * FIX["sums"]["dW1_abs"]
    assert abs(float(dw2.double().abs().sum()) - FIX["sums"]["dW2_abs"]) < 1e-3 * FIX["sums"]["dW2_abs"]


def test_oracle_reproduces_fixture():
    cfg = CONFIGS["c1"]
    t = make_inputs(cfg, seed=0)
    x, p = t["x"].clone().requires_grad_(), t["p"].clone().requires_grad_()
    W1, W2 = t["W1"].clone().requires_grad_(), t["W2"].clone().requires_grad_()
    y = oracle.naive_expert_forward(x, p, t["experts"], W1, W2, torch.nn.GELU())
    g = torch.autograd.grad(y, [x, p, W1, W2], t["dy"])
    _check(y.detach(), *g, oracle.route_ref(t["experts"], cfg.E), 1e-5)


@pytest.mark.gpu
def test_hip_path_reproduces_fixture():
    from scattermoe_amd import flatten_sort_count
    from scattermoe_amd.mlp import MLP
    cfg = CONFIGS["c1"]
    t = make_inputs(cfg, seed=0)
    dev = "cuda:0"
    m = MLP(cfg.d, cfg.f, cfg.E, cfg.k, activation=torch.nn.GELU()).to(dev)
    with torch.no_grad():
        m.experts.weight.copy_(t["W1"]); m.output_experts.weight.copy_(t["W2"])
    x, p = t["x"].to(dev).requires_grad_(), t["p"].to(dev).requires_grad_()
    y = m(x, p, t["experts"].to(dev))
    g = torch.autograd.grad(y, [x, p, m.experts.weight, m.output_experts.weight], t["dy"].to(dev))
    _check(y.detach(), *g, flatten_sort_count(t["experts"].to(dev), cfg.E), 1e-4)
