"""Seeded synthetic inputs for the benchmark configurations (generated on CPU in fp32, then cast/moved,
so CPU and GPU runs see identical values).  Draw order: router logits, X, W1, W2, [b1, b2], dY."""
from dataclasses import dataclass

import torch


@dataclass
class Config:
    name: str
    T: int
    d: int
    f: int
    E: int
    k: int
    glu: bool
    bias: bool = False
    zipf_beta: float = 0.0
    dtype: torch.dtype = torch.bfloat16


CONFIGS = {
    "c1": Config("c1", 256, 128, 256, 8, 2, glu=False, dtype=torch.float32),
    "c2": Config("c2", 16384, 4096, 14336, 8, 2, glu=True),
    "c3": Config("c3", 8192, 2880, 2880, 32, 4, glu=True, bias=True, zipf_beta=1.5),
    "c4": Config("c4", 32768, 2048, 768, 128, 8, glu=True),
}


def scaled(cfg, T=None, d=None, f=None):
    return Config(cfg.name + "_s", T or cfg.T, d or cfg.d, f or cfg.f, cfg.E, cfg.k, cfg.glu, cfg.bias,
                  cfg.zipf_beta, cfg.dtype)


def make_inputs(cfg, seed=0, weights=True):
    g = torch.Generator("cpu").manual_seed(seed)
    n1 = (2 if cfg.glu else 1) * cfg.f
    logits = torch.randn(cfg.T, cfg.E, generator=g)
    if cfg.zipf_beta:
        logits = logits + cfg.zipf_beta * (-1.2 * torch.log(torch.arange(1, cfg.E + 1, dtype=torch.float32)))
    probs = torch.softmax(logits.float(), dim=-1)
    p, experts = torch.topk(probs, cfg.k)
    p = p / p.sum(-1, keepdim=True)
    out = {"p": p, "experts": experts}
    out["x"] = torch.randn(cfg.T, cfg.d, generator=g)
    if weights:
        out["W1"] = torch.randn(cfg.E, n1, cfg.d, generator=g) * 0.02
        out["W2"] = torch.randn(cfg.E, cfg.d, cfg.f, generator=g) * 0.02
        if cfg.bias:
            out["b1"] = torch.randn(cfg.E, n1, generator=g) * 0.02
            out["b2"] = torch.randn(cfg.E, cfg.d, generator=g) * 0.02
    out["dy"] = torch.randn(cfg.T, cfg.d, generator=g)
    return out


def make_module(cfg, device, seed=1):
    """The module of a configuration with weights (and biases) drawn N(0, 0.02) on `device` from a device generator:
    the draw that the full-shape GPU tests and bench.py share (drawing up to 5.6e9 normal numbers on the host takes
    longer than everything else they do)."""
    from torch import nn
    from scattermoe_amd.mlp import GLUMLP, MLP
    g = torch.Generator(device=device).manual_seed(seed)
    with torch.device(device):
        if cfg.glu:
            m = GLUMLP(cfg.d, cfg.f, cfg.E, cfg.k, bias=cfg.bias).to(cfg.dtype)
        else:
            m = MLP(cfg.d, cfg.f, cfg.E, cfg.k, bias=cfg.bias, activation=nn.GELU()).to(cfg.dtype)
    with torch.no_grad():
        for prm in m.parameters():
            prm.copy_((torch.randn(prm.shape, generator=g, device=device) * 0.02).to(cfg.dtype))
    return m
