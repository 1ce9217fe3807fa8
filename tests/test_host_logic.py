"""Host-side logic on CPU: the autograd dataflow of ParallelLinear / MLP / GLUMLP with the device launch
layer replaced by the oracle's kernel models (fixture `cpu_backend`).  Compared with the naive MoE MLP,
the quantities and the 1e-4 fp32 bound of the reference test (tests/test_mlp.py:66-87)."""
import pytest
import torch
from torch import nn

import oracle


def _case(T, d, h, E, k, bias, glu, seed=0):
    from scattermoe_amd.mlp import MLP, GLUMLP
    torch.manual_seed(seed)
    logits = torch.randn(T, E)
    w = torch.softmax(logits, -1)
    p, experts = torch.topk(w, k)
    p = p.clone().requires_grad_()
    x = torch.randn(T, d, requires_grad=True)
    dy = torch.randn(T, d)
    m = (GLUMLP(d, h, E, k, bias=bias) if glu else MLP(d, h, E, k, bias=bias, activation=nn.GELU()))
    if bias:
        nn.init.normal_(m.experts.bias, std=0.02)
        nn.init.normal_(m.output_experts.bias, std=0.02)
    return m, x, p, experts, dy


@pytest.mark.parametrize("glu", [False, True])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("T,d,k", [(1, 128, 2), (33, 100, 3), (64, 96, 4)])
def test_mlp_matches_naive(cpu_backend, T, d, k, bias, glu):
    E, h = 8, (4 * d) // k
    m, x, p, experts, dy = _case(T, d, h, E, k, bias, glu)
    params = [x, p, m.experts.weight, m.output_experts.weight]
    if bias:
        params += [m.experts.bias, m.output_experts.bias]
    y = m(x, p, experts)
    got = torch.autograd.grad(y, params, dy)
    y_ref = oracle.naive_module_forward(m, x, p, experts, per_token=(T <= 33))
    want = torch.autograd.grad(y_ref, params, dy)
    assert (y - y_ref).abs().max() < 1e-4
    for a, b in zip(got, want):
        assert a.shape == b.shape
        assert (a - b).abs().max() < 1e-4


def test_weight_grad_is_contiguous_in_parameter_layout(cpu_backend):
    m, x, p, experts, dy = _case(16, 32, 24, 4, 2, True, False)
    m(x, p, experts).backward(dy)
    assert m.experts.weight.grad.is_contiguous() and m.experts.weight.grad.shape == m.experts.weight.shape
    assert m.output_experts.bias.grad.shape == m.output_experts.bias.shape


@pytest.mark.parametrize("grouped_in,grouped_out", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("use_gates", [False, True])
def test_parallel_linear_all_layouts(cpu_backend, grouped_in, grouped_out, use_gates):
    """parallel_linear against a per-row dense formulation, incl. the k == 1 and ungrouped branches the
    reference never tests."""
    import scattermoe_amd as sm
    if use_gates and grouped_out:
        pytest.skip("gates combine slot-ordered outputs")
    torch.manual_seed(1)
    T, E, k, K, N = 10, 4, 2, 6, 5
    experts = torch.topk(torch.randn(T, E), k).indices
    eid, idx, off = sm.flatten_sort_count(experts, E)
    W = torch.randn(E, K, N, requires_grad=True)
    b = torch.randn(E, N, requires_grad=True)
    gates = torch.rand(T, k, requires_grad=True) if use_gates else None
    x_rows = T * k if grouped_in else T
    x = torch.randn(x_rows, K, requires_grad=True)
    fan = 1 if grouped_in else k
    y = sm.parallel_linear(x, W, fan, eid, idx, off, expert_biases=b, gates=gates,
                           grouped_in=grouped_in, grouped_out=grouped_out)
    # dense statement: row n (sorted order) uses expert eid[n], source row n | idx[n]//k, target n | idx[n]
    rows = torch.arange(T * k)
    src = rows if grouped_in else idx // k
    per_row = torch.einsum("nk,nkj->nj", x[src], W[eid]) + b[eid]
    dst = rows if grouped_out else idx
    y_ref = torch.zeros(T * k, N).index_add(0, dst, per_row)
    if use_gates:
        y_ref = (y_ref.view(T, k, N) * gates.unsqueeze(-1)).sum(1)
    assert torch.allclose(y, y_ref, atol=1e-5)
    dy = torch.randn_like(y)
    inputs = [x, W, b] + ([gates] if use_gates else [])
    for a, c in zip(torch.autograd.grad(y, inputs, dy), torch.autograd.grad(y_ref, inputs, dy)):
        assert torch.allclose(a, c, atol=1e-5)


def test_needs_input_grad_skips(cpu_backend):
    import scattermoe_amd as sm
    torch.manual_seed(2)
    T, E, k, K, N = 6, 3, 2, 4, 4
    experts = torch.topk(torch.randn(T, E), k).indices
    eid, idx, off = sm.flatten_sort_count(experts, E)
    x = torch.randn(T, K, requires_grad=True)
    W = torch.randn(E, K, N)                      # frozen experts: only dX flows
    y = sm.parallel_linear(x, W, k, eid, idx, off)
    (gx,) = torch.autograd.grad(y, [x], torch.ones_like(y))
    want = torch.zeros(T, K).index_add(0, idx // k, torch.einsum("nj,nkj->nk", torch.ones(T * k, N), W[eid]))
    assert torch.allclose(gx, want, atol=1e-5)


def test_api_surface_and_errors(cpu_backend):
    import scattermoe_amd as sm
    from scattermoe_amd.kernels import ops
    for name in ("flatten_sort_count", "parallel_linear", "ParallelExperts", "parallel_experts", "kernels", "mlp"):
        assert hasattr(sm, name)
    assert ops.BLOCK_M == 128 and ops.ALLOW_TF32 is True
    for op in ("bincount", "scatter2scatter", "groupXtY", "group"):
        assert hasattr(torch.ops.scattermoe, op)
    m = sm.mlp.MLP(8, 16, 4, 9, activation=nn.Identity())
    assert m.top_k == 4                                            # top_k is clipped to the expert count
    assert set(sm.mlp.GLUMLP(8, 16, 4, 2, bias=True).state_dict()) == {
        "experts.weight", "experts.bias", "output_experts.weight", "output_experts.bias"}
    assert sm.mlp.GLUMLP(8, 16, 4, 2).experts.weight.shape == (4, 32, 8)
    assert repr(sm.ParallelExperts(2, 3, 5)) == "ParallelExperts(num_experts=2, input_size=3, output_size=5)"
    eid, idx, off = sm.flatten_sort_count(torch.tensor([[0, 1], [1, 0]]), 2)
    with pytest.raises(AssertionError):                            # row count must be X.size(0) * k
        ops.scatter2scatter(torch.randn(3, 4), torch.randn(2, 4, 4), eid, idx, 2)
    with pytest.raises(AssertionError):
        ops.group(torch.randn(3, 4), idx, fan_out=2)
    with pytest.raises(AssertionError):
        ops.scatter2scatter(torch.randn(2, 4), torch.randn(2, 4, 4), eid, idx, 2, out=torch.empty(4, 5))


def test_mixture_of_lora_module_prints_like_the_reference():
    """The module of the reference's example (examples/molora.py:5-24) and the text it prints there."""
    import scattermoe_amd as sm
    m = sm.mlp.MLP(input_size=1024, hidden_size=128, num_experts=16, top_k=2, activation=nn.Identity())
    assert repr(m) == ("MLP(\n  k=2\n"
                       "  (experts): ParallelExperts(num_experts=16, input_size=1024, output_size=128)\n"
                       "  (output_experts): ParallelExperts(num_experts=16, input_size=128, output_size=1024)\n"
                       "  (activation): Identity()\n)")


def test_product_path_refuses_cpu_tensors():
    """Without the test double the launch layer is the HIP library and must not silently run on CPU."""
    import scattermoe_amd as sm
    with pytest.raises(RuntimeError, match="ROCm GPU only"):
        sm.flatten_sort_count(torch.tensor([[0, 1]]), 2)


@pytest.mark.parametrize("glu", [False, True])
def test_second_backward_over_a_consumed_graph_is_refused(cpu_backend, glu):
    """Without gate gradients, backward reuses the saved expert-output buffer for the grouped output gradient.  A
    second backward over the same graph must not silently read the overwritten buffer: like the reference, whose
    `group` op declares the buffer as mutated (scattermoe/kernels/ops.py:389), it has to raise."""
    m, x, p, experts, dy = _case(16, 32, 24, 4, 2, False, glu)
    y = m(x, p.detach(), experts)
    y.backward(dy, retain_graph=True)
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        y.backward(dy)


@pytest.mark.parametrize("glu", [False, True])
def test_second_backward_with_gate_gradients_repeats_the_first(cpu_backend, glu):
    """With gate gradients the grouped output gradient gets a buffer of its own (it is written in the pass that
    still reads the expert outputs), so the saved tensors stay intact and a retained graph can be walked again."""
    m, x, p, experts, dy = _case(16, 32, 24, 4, 2, False, glu)
    y = m(x, p, experts)
    first = torch.autograd.grad(y, [x, p, m.experts.weight], dy, retain_graph=True)
    second = torch.autograd.grad(y, [x, p, m.experts.weight], dy)
    for a, b in zip(first, second):
        assert torch.equal(a, b)


def test_slot_sum_is_the_gateless_combine(cpu_backend):
    ops = cpu_backend
    y = torch.randn(5 * 3, 7)
    assert torch.allclose(ops.slot_sum(y, 5, 3), y.view(5, 3, 7).sum(1), atol=1e-6)
    assert ops.slot_sum(y, 15, 1) is y


def test_stale_library_is_refused(monkeypatch):
    """The loader compares the digest compiled into the library with the sources beside it."""
    import scattermoe_amd._C as C
    from scattermoe_amd import _build
    assert C.source_hash() == _build.source_hash()
    monkeypatch.setattr(C, "_lib", None)
    monkeypatch.setattr(_build, "source_hash", lambda: "0" * 16)
    with pytest.raises(RuntimeError, match="stale"):
        C.load()
