"""GPU parity of the router front end (softmax -> top-k -> renormalise in one launch) against the CPU oracle:
expert ids bit-exact wherever the two largest candidates differ by more than rounding, weights to 1e-5."""
import pytest
import torch

import oracle
from scattermoe_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _check(logits, k, renorm):
    w, i = ops.topk_softmax(logits.to(DEV), k, renorm)
    assert w.dtype == torch.float32 and i.dtype == torch.int64 and w.shape == i.shape == (logits.size(0), k)
    rw, ri = oracle.topk_softmax_ref(logits, k, renorm)
    w, i = w.cpu(), i.cpu()
    same = i == ri
    if not bool(same.all()):
        # a swap is only legitimate between probabilities that are equal to rounding
        p = torch.softmax(logits.float(), -1)
        assert torch.allclose(p.gather(1, i), p.gather(1, ri), rtol=1e-6, atol=0)
    torch.testing.assert_close(w, rw, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("T,E,k", [(1, 8, 2), (3, 1, 1), (257, 8, 2), (16384, 8, 2), (4096, 32, 4), (1000, 128, 8),
                                   (333, 300, 3), (64, 512, 64), (100, 4, 4), (70, 64, 1), (70, 65, 5)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("renorm", [True, False])
def test_topk_softmax(T, E, k, dtype, renorm):
    g = torch.Generator().manual_seed(T + 7 * E + k)
    logits = (torch.randn(T, E, generator=g) * 2.5).to(dtype)
    if dtype is not torch.float32:
        # 16-bit logits collide often; make every row's values distinct so that the order is fixed
        logits = (torch.rand(T, E, generator=g).argsort(-1).float() * (8.0 / E) - 4.0).to(dtype)
        if E > 256:
            logits = torch.rand(T, E, generator=g).argsort(-1).float().sub(256).div(16).to(dtype)
    _check(logits, k, renorm)


def test_topk_softmax_ties_strides_and_errors():
    w, i = ops.topk_softmax(torch.zeros(5, 70, device=DEV), 4, False)
    assert i.tolist() == [[0, 1, 2, 3]] * 5 and torch.allclose(w.cpu(), torch.full((5, 4), 1 / 70))
    logits = torch.tensor([[0.0, 3.0, 3.0, -1.0, 3.0]], device=DEV)
    assert ops.topk_softmax(logits, 3)[1].tolist() == [[1, 2, 4]]
    big = torch.randn(40, 24, generator=torch.Generator().manual_seed(3))
    view = big[:, ::3]                                      # strided columns
    w1, i1 = ops.topk_softmax(big.to(DEV)[:, ::3], 2)
    rw, ri = oracle.topk_softmax_ref(view, 2)
    assert torch.equal(i1.cpu(), ri) and torch.allclose(w1.cpu(), rw, rtol=1e-5)
    tr = big.t().contiguous().to(DEV).t()                  # token stride 1
    w2, i2 = ops.topk_softmax(tr, 2)
    rw, ri = oracle.topk_softmax_ref(big, 2)
    assert torch.equal(i2.cpu(), ri) and torch.allclose(w2.cpu(), rw, rtol=1e-5)
    w0, i0 = ops.topk_softmax(torch.empty(0, 8, device=DEV), 2)
    assert w0.shape == i0.shape == (0, 2)
    with pytest.raises(ValueError):
        ops.topk_softmax(torch.zeros(4, 8, device=DEV), 9)
    with pytest.raises(RuntimeError):
        ops.topk_softmax(torch.zeros(4, 600, device=DEV), 2)
    # extreme logits: no overflow
    w, i = ops.topk_softmax(torch.tensor([[1e4, -1e4, 0.0, 9990.0]], device=DEV), 2, False)
    assert i.tolist() == [[0, 3]] and abs(float(w[0, 0]) - 1.0) < 1e-4


@pytest.mark.parametrize("renorm", [True, False])
def test_topk_softmax_gradient(renorm):
    g = torch.Generator().manual_seed(11)
    logits = torch.randn(50, 16, generator=g)
    d_w = torch.randn(50, 4, generator=g)
    a = logits.clone().to(DEV).requires_grad_(True)
    w, i = ops.topk_softmax(a, 4, renorm)
    w.backward(d_w.to(DEV))
    b = logits.clone().double().requires_grad_(True)
    p = torch.softmax(b, -1)
    tw, ti = torch.topk(p, 4)
    if renorm:
        tw = tw / tw.sum(-1, keepdim=True)
    tw.backward(d_w.double())
    assert torch.equal(i.cpu(), ti)
    torch.testing.assert_close(a.grad.cpu().double(), b.grad, rtol=1e-4, atol=1e-6)


def test_router_feeds_the_mlp():
    """The front end's outputs are what GLUMLP takes: same result as routing with torch ops."""
    from scattermoe_amd.mlp import GLUMLP
    torch.manual_seed(5)
    m = GLUMLP(64, 96, 8, 2).to(DEV)
    x = torch.randn(300, 64, device=DEV)
    logits = torch.randn(300, 8, device=DEV)
    w, i = ops.topk_softmax(logits, 2)
    tw, ti = torch.topk(torch.softmax(logits.float(), -1), 2)
    tw = tw / tw.sum(-1, keepdim=True)
    assert torch.equal(i, ti)
    torch.testing.assert_close(m(x, w, i), m(x, tw, ti), rtol=1e-5, atol=1e-6)


def test_unusable_logits_still_give_valid_experts():
    """NaN logits never win, rows without any usable logit are routed as all-equal, +inf is the maximum: every id
    is a valid expert and every weight finite, so no row of the layer output is left unwritten downstream."""
    E, k = 8, 2
    nan, inf = float("nan"), float("inf")
    logits = torch.tensor([[0.0, nan, 1.0, 2.0, nan, -1.0, 0.5, 0.25],
                           [nan] * 8,
                           [-inf] * 8,
                           [0.0, inf, 1.0, 2.0, 3.0, 4.0, 5.0, 6.0],
                           [nan, nan, nan, nan, nan, nan, nan, 3.0]])
    w, i = ops.topk_softmax(logits.to(DEV), k, True)
    w, i = w.cpu(), i.cpu()
    assert bool(((i >= 0) & (i < E)).all()) and bool(torch.isfinite(w).all())
    assert i[0].tolist() == [3, 2] and i[1].tolist() == [0, 1] and i[2].tolist() == [0, 1] and i[3, 0].item() == 1
    assert i[4, 0].item() == 7 and abs(w[4, 0].item() - 1.0) < 1e-6
    torch.testing.assert_close(w.sum(-1), torch.ones(5))
    rw, ri = oracle.topk_softmax_ref(logits[:1].nan_to_num(nan=-inf), k, True)
    torch.testing.assert_close(w[:1], rw, rtol=1e-5, atol=1e-7)
