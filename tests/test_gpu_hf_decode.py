"""GPU parity of the Hugging Face injection and of the decode regime (BASELINE config 5)."""
import pytest
import torch

import oracle
from scattermoe_amd.kernels import ops
from scattermoe_amd.kernels.single import single2scatter

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _close(got, want, rtol, atol):
    got, want = got.detach().float().cpu(), want.detach().float()
    bound = atol * max(1.0, want.abs().max().item()) + rtol * want.abs()
    err = (got - want).abs()
    assert bool((err <= bound).all()), "max err %g" % err.max()


@pytest.mark.parametrize("dtype,rtol,atol", [(torch.float32, 1e-4, 1e-5), (torch.bfloat16, 2e-2, 1e-2)])
def test_gpt_oss_patched_forward_backward(dtype, rtol, atol):
    transformers = pytest.importorskip("transformers")
    from transformers import GptOssConfig
    import transformers.models.gpt_oss.modeling_gpt_oss as M
    from scattermoe_amd.utils import replace_moe as src
    T, E, k, d, f = 300, 8, 4, 64, 96
    g = torch.Generator().manual_seed(0)
    ref = M.GptOssExperts(GptOssConfig(hidden_size=d, intermediate_size=f, num_local_experts=E, num_experts_per_tok=k))
    with torch.no_grad():
        for prm in ref.parameters():
            prm.copy_((torch.randn(prm.shape, generator=g) * 0.2).to(dtype).float())
    x = torch.randn(T, d, generator=g).to(dtype)
    top, index = torch.topk(torch.randn(T, E, generator=g), k)
    weights = torch.softmax(top, -1).to(dtype)

    xc = x.float().requires_grad_()
    wc = weights.float().requires_grad_()
    want = oracle.naive_expert_forward(xc, wc, index, ref.gate_up_proj.transpose(1, 2), ref.down_proj.transpose(1, 2),
                                       oracle.gpt_oss_glu(ref.alpha, ref.limit), ref.gate_up_proj_bias, ref.down_proj_bias)
    gw = torch.autograd.grad(want, [xc, wc, ref.gate_up_proj, ref.down_proj, ref.gate_up_proj_bias, ref.down_proj_bias],
                             torch.ones_like(want))

    mod = M.GptOssExperts(GptOssConfig(hidden_size=d, intermediate_size=f, num_local_experts=E, num_experts_per_tok=k))
    mod.load_state_dict(ref.state_dict())
    mod = mod.to(DEV).to(dtype)
    xg = x.to(DEV).requires_grad_()
    wg = weights.to(DEV).requires_grad_()
    got = src.gpt_oss_forward(mod, xg, index.to(DEV), wg)
    gg = torch.autograd.grad(got, [xg, wg, mod.gate_up_proj, mod.down_proj, mod.gate_up_proj_bias, mod.down_proj_bias],
                             torch.ones_like(got))
    _close(got, want, rtol, atol)
    for a, b in zip(gg, gw):
        _close(a, b, rtol, atol)
    # weight gradients come back in the layout of the (E, in, out) parameters: nothing left to transpose
    assert gg[2].is_contiguous() and gg[3].is_contiguous()


def test_hf_experts_gate_first_glu():
    from scattermoe_amd.utils import replace_moe as src
    T, E, k, d, f = 257, 8, 2, 128, 192
    g = torch.Generator().manual_seed(1)

    class Experts(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.num_experts = E
            self.gate_up_proj = torch.nn.Parameter(torch.randn(E, 2 * f, d, generator=g) * 0.1)
            self.down_proj = torch.nn.Parameter(torch.randn(E, d, f, generator=g) * 0.1)
            self.act_fn = torch.nn.SiLU()

    m = Experts()
    x = torch.randn(T, d, generator=g)
    top, index = torch.topk(torch.randn(T, E, generator=g), k)
    weights = torch.softmax(top, -1)
    gate, up = m.gate_up_proj.detach().chunk(2, dim=1)
    want = oracle.naive_expert_forward(x, weights, index, torch.cat([up, gate], 1), m.down_proj.detach(),
                                       oracle.glu(torch.nn.functional.silu))
    mg = Experts().to(DEV)
    mg.load_state_dict(m.state_dict())
    got = src.experts_forward(mg, x.to(DEV), index.to(DEV), weights.to(DEV))
    _close(got, want, 1e-4, 1e-5)
    # decode sizes in bf16 without autograd take the two-launch step: same bits as the general path, close to fp32
    mh = mg.to(torch.bfloat16)
    xs, ws, ix = x[:3].to(DEV).bfloat16(), weights[:3].to(DEV).bfloat16(), index[:3].to(DEV)
    general = src.experts_forward(mh, xs, ix, ws)
    with torch.no_grad():
        step = src.experts_forward(mh, xs, ix, ws)
    assert torch.equal(step, general.detach())
    _close(step, want[:3], 3e-2, 2e-2)


@pytest.mark.parametrize("T", [1, 8, 64, 256])
def test_decode_regime_matches_oracle(T):
    """Mixtral-shaped decode at reduced width: T tokens, uniform random routing, forward only."""
    E, k, d, f = 8, 2, 512, 1024
    g = torch.Generator().manual_seed(T)
    experts = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    x = torch.randn(T, d, generator=g).bfloat16()
    W1 = (torch.randn(E, 2 * f, d, generator=g) * 0.05).bfloat16()
    eid, idx, off = oracle.route_ref(experts, E)
    want = oracle.scatter2scatter_ref(x.float(), W1.permute(0, 2, 1).float(), eid, idx, k, None, False, True)
    r = ops.route(experts.to(DEV), E)
    assert all(torch.equal(a.cpu(), b) for a, b in zip(r, (eid, idx, off)))
    got = ops.scatter2scatter(x.to(DEV), W1.to(DEV).permute(0, 2, 1), r[0], r[1], k, y_grouped=True, expert_offsets=r[2])
    _close(got, want, 2e-2, 1e-2)


def test_single2scatter_gpu():
    g = torch.Generator().manual_seed(2)
    E, K, N, k = 8, 256, 384, 2
    W = (torch.randn(E, K, N, generator=g) * 0.1).bfloat16()
    experts = torch.tensor([[5, 2]])
    for rows in (1, k):
        x = torch.randn(rows, K, generator=g).bfloat16()
        want = torch.stack([x[j if rows == k else 0].float() @ W[e].float() for j, e in enumerate(experts[0])])
        got = single2scatter(x.to(DEV), W.to(DEV), experts.to(DEV))
        _close(got, want, 2e-2, 1e-2)


@pytest.mark.parametrize("T", [1, 4, 40])
def test_decode_forward_replays_from_a_hip_graph(T):
    """The library allocates, clears and synchronises nothing, so a whole module forward captures into a HIP graph.
    Every replay (new inputs written into the static buffers, eager work and synchronisations in between) must
    reproduce the eager result bit for bit.  T = 1 and 4 run the row-dot kernels, T = 40 the ring tiles."""
    from scattermoe_amd.mlp import GLUMLP
    from scattermoe_amd.kernels.ops import topk_softmax
    E, k, d, f = 8, 2, 256, 384
    torch.manual_seed(7)
    with torch.device(DEV):
        m = GLUMLP(d, f, E, k).to(torch.bfloat16)
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, d, generator=g).to(torch.bfloat16).to(DEV)
    logits = torch.randn(T, E, generator=g).to(DEV)

    def step(xx, ll):
        w, i = topk_softmax(ll, k)
        return m(xx, w.to(torch.bfloat16), i)

    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                step(x, logits)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_static = step(x, logits)
        for r in range(4):
            x.copy_(torch.randn(T, d, generator=g).to(torch.bfloat16))
            logits.copy_(torch.randn(T, E, generator=g))
            graph.replay()
            torch.cuda.synchronize()
            got = y_static.clone()
            want = step(x, logits)                       # eager work between the replays
            torch.cuda.synchronize()
            assert torch.equal(got, want), "replay %d differs from the eager result" % r


def test_tiny_mixtral_model_end_to_end():
    """A whole (tiny, randomly initialised) Hugging Face Mixtral with its experts class patched: logits and the
    gradient of an expert weight against the unpatched model (HF's own per-expert loop), float32."""
    transformers = pytest.importorskip("transformers")
    from transformers import MixtralConfig, MixtralForCausalLM
    import transformers.models.mixtral.modeling_mixtral as MX
    from scattermoe_amd.utils import replace_moe as src
    if not hasattr(MX, "MixtralExperts"):
        pytest.skip("transformers without MixtralExperts")
    cfg = MixtralConfig(vocab_size=128, hidden_size=64, intermediate_size=96, num_hidden_layers=2,
                        num_attention_heads=4, num_key_value_heads=2, num_local_experts=4, num_experts_per_tok=2,
                        max_position_embeddings=64, hidden_act="silu")
    torch.manual_seed(0)
    model = MixtralForCausalLM(cfg).to(DEV)
    ids = torch.randint(0, 128, (2, 17), generator=torch.Generator().manual_seed(1)).to(DEV)
    original = MX.MixtralExperts.forward
    try:
        want = model(ids).logits
        want.float().pow(2).mean().backward()
        w_ref = model.model.layers[0].mlp.experts.gate_up_proj.grad.clone()
        model.zero_grad()
        src.patch_experts_class(MX.MixtralExperts)
        got = model(ids).logits
        assert MX.MixtralExperts.forward is src.experts_forward          # the lazy patch has replaced itself
        got.float().pow(2).mean().backward()
        w_got = model.model.layers[0].mlp.experts.gate_up_proj.grad
        torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(w_got, w_ref, rtol=1e-3, atol=1e-6)
        with torch.no_grad():                                            # one new token: the decode step kernels
            step = model(ids[:, :1]).logits
        MX.MixtralExperts.forward = original
        with torch.no_grad():
            torch.testing.assert_close(step, model(ids[:, :1]).logits, rtol=1e-4, atol=1e-4)
    finally:
        MX.MixtralExperts.forward = original


def test_tiny_gpt_oss_model_end_to_end():
    """A whole tiny gpt-oss with the import-time patch of its experts against the forward the class had before."""
    transformers = pytest.importorskip("transformers")
    from transformers import GptOssConfig, GptOssForCausalLM
    import transformers.models.gpt_oss.modeling_gpt_oss as M
    from scattermoe_amd.utils import replace_moe as src
    patched = M.GptOssExperts.forward
    original = getattr(patched, "__original__", None)
    if original is None:
        pytest.skip("GptOssExperts was not patched in this process")
    cfg = GptOssConfig(vocab_size=128, hidden_size=64, intermediate_size=64, num_hidden_layers=2, head_dim=16,
                       num_attention_heads=4, num_key_value_heads=2, num_local_experts=4, num_experts_per_tok=2,
                       max_position_embeddings=64, sliding_window=16, layer_types=["sliding_attention", "full_attention"])
    torch.manual_seed(0)
    model = GptOssForCausalLM(cfg).to(DEV)
    with torch.no_grad():
        for n, prm in model.named_parameters():
            if "experts" in n:
                prm.normal_(0, 0.1)
    ids = torch.randint(0, 128, (2, 9), generator=torch.Generator().manual_seed(2)).to(DEV)
    try:
        got = model(ids).logits
        got.float().pow(2).mean().backward()
        g_got = model.model.layers[1].mlp.experts.down_proj.grad.clone()
        model.zero_grad()
        M.GptOssExperts.forward = original
        want = model(ids).logits
        want.float().pow(2).mean().backward()
        g_want = model.model.layers[1].mlp.experts.down_proj.grad
        torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(g_got, g_want, rtol=1e-3, atol=1e-6)
    finally:
        M.GptOssExperts.forward = patched


def _grads(out, params, seed=9):
    dy = torch.randn(out.shape, generator=torch.Generator().manual_seed(seed)).to(out.dtype).to(out.device)
    return torch.autograd.grad(out, params, dy)


@pytest.mark.parametrize("dtype,rtol,atol", [(torch.float32, 1e-4, 1e-5), (torch.bfloat16, 2e-2, 1e-2)])
def test_granite_block_on_gpu_against_hf_original(dtype, rtol, atol):
    """`granite_moe_forward` (reference scattermoe/utils/replace_moe.py:60-95) on the GraniteMoeHybridMoE block of
    the installed transformers (router + experts module), forward and backward, against the block's own original
    forward (Hugging Face's per-expert loop) run in float32 on the CPU from the same parameters."""
    pytest.importorskip("transformers")
    from transformers import GraniteMoeHybridConfig
    import transformers.models.granitemoehybrid.modeling_granitemoehybrid as GR
    from scattermoe_amd.utils import replace_moe as src
    d, f, E, k = 128, 192, 8, 2
    cfg = GraniteMoeHybridConfig(hidden_size=d, intermediate_size=f, num_local_experts=E, num_experts_per_tok=k,
                                 hidden_act="silu", mamba_n_heads=4, mamba_expand=2)
    original = getattr(GR.GraniteMoeHybridMoE.forward, "__original__", None) or GR.GraniteMoeHybridMoE.forward
    assert original is not src.granite_moe_forward
    g = torch.Generator().manual_seed(4)
    ref = GR.GraniteMoeHybridMoE(cfg)
    with torch.no_grad():
        for prm in ref.parameters():
            prm.copy_((torch.randn(prm.shape, generator=g) * 0.1).to(dtype).float())
    blk = GR.GraniteMoeHybridMoE(cfg)
    blk.load_state_dict(ref.state_dict())
    blk = blk.to(DEV).to(dtype)
    xin = torch.randn(3, 50, d, generator=g).to(dtype)
    xc = xin.float().requires_grad_()
    want = original(ref, xc)
    xg = xin.to(DEV).requires_grad_()
    got = src.granite_moe_forward(blk, xg)
    assert got.shape == (3, 50, d) and got.dtype == dtype
    # the comparison needs both sides to route alike: in bf16 the router's matmul may flip near-ties
    same = torch.equal(blk.router(xg.detach().reshape(-1, d))[0].cpu(), ref.router(xc.detach().reshape(-1, d))[0])
    if dtype is torch.float32:
        assert same
    if same:
        _close(got, want, rtol, atol)
        names = [n for n, _ in ref.named_parameters()]
        for n, a, b in zip(["x"] + names, _grads(got, [xg] + list(blk.parameters())),
                           _grads(want, [xc] + list(ref.parameters()))):
            _close(a, b, rtol, atol)
    else:
        rows = (blk.router(xg.detach().reshape(-1, d))[0].cpu() == ref.router(xc.detach().reshape(-1, d))[0]).all(-1)
        assert float(rows.float().mean()) > 0.9
        _close(got.reshape(-1, d)[rows.to(DEV)], want.reshape(-1, d)[rows], rtol, atol)


@pytest.mark.parametrize("dtype,rtol,atol", [(torch.float32, 1e-4, 1e-5), (torch.bfloat16, 2e-2, 1e-2)])
def test_granite_block_of_transformers_4_on_gpu(dtype, rtol, atol):
    """The block layout the reference patched (`router.layer`, `router.top_k`, `input_linear.weight`,
    `output_linear.weight`, `activation`; replace_moe.py:63-93), which transformers 5.x no longer ships: a stand-in
    with those attributes, router front end (softmax -> top-k -> renormalise in one launch) included, against the
    oracle's per-expert form fed with `oracle.topk_softmax_ref`."""
    from types import SimpleNamespace
    from scattermoe_amd.utils import replace_moe as src
    E, k, d, f = 8, 2, 128, 192
    g = torch.Generator().manual_seed(8)
    lw = (torch.randn(E, d, generator=g) * 0.5).to(dtype)
    w_in = (torch.randn(E, 2 * f, d, generator=g) * 0.1).to(dtype)
    w_out = (torch.randn(E, d, f, generator=g) * 0.1).to(dtype)
    xin = torch.randn(4, 33, d, generator=g).to(dtype)
    layer = torch.nn.Linear(d, E, bias=False).to(DEV).to(dtype)
    with torch.no_grad():
        layer.weight.copy_(lw)
    p_in = torch.nn.Parameter(w_in.to(DEV))
    p_out = torch.nn.Parameter(w_out.to(DEV))
    blk = SimpleNamespace(router=SimpleNamespace(layer=layer, top_k=k, num_experts=E),
                          input_linear=SimpleNamespace(weight=p_in), output_linear=SimpleNamespace(weight=p_out),
                          activation=torch.nn.SiLU())
    xg = xin.to(DEV).requires_grad_()
    got, logits = src.granite_moe_forward(blk, xg)
    assert got.shape == xin.shape and logits.shape == (4 * 33, E)
    # oracle on the router logits the GPU produced (so that both sides route alike), weights rounded like the block's
    w, sel = oracle.topk_softmax_ref(logits.detach().float().cpu(), k, True)
    xc = xin.float().reshape(-1, d).requires_grad_()
    gate, up = w_in.float().chunk(2, dim=1)
    W1 = torch.cat([up, gate], 1).requires_grad_()          # the oracle's gated unit activates the SECOND half
    W2 = w_out.float().requires_grad_()
    want = oracle.naive_expert_forward(xc, w.to(dtype).float(), sel, W1, W2, oracle.glu(torch.nn.functional.silu))
    _close(got.reshape(-1, d), want, rtol, atol)
    dy = torch.randn(want.shape, generator=g).to(dtype)
    gx, gin, gout = torch.autograd.grad(got, [xg, p_in, p_out], dy.to(DEV).view(got.shape))
    # the oracle side keeps the routing weights constant, so compare only what does not flow through the router
    wx, w1g, w2g = torch.autograd.grad(want, [xc, W1, W2], dy.float())
    up_g, gate_g = w1g.chunk(2, dim=1)
    _close(gin, torch.cat([gate_g, up_g], 1), rtol, atol)
    _close(gout, w2g, rtol, atol)
