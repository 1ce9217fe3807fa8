"""Writes tests/golden/c1_seed0.json: BASELINE config 1 (T=256, d=128, f=256, E=8, k=2, GELU, fp32, seed 0)
evaluated by the CPU oracle (oracle/naive_moe.py) in this repository — checksums of the inputs, the routing triple
in full, and a few rows / checksums of Y, dX, dg, dW1, dW2.  The reference keeps no stored vectors of its own
(tests/test_mlp.py draws unseeded inputs), so this fixture records the oracle's answer for regression use.

    python tests/golden/make_c1_fixture.py
"""
import hashlib
import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import oracle  # noqa: E402
from _inputs import CONFIGS, make_inputs  # noqa: E402


def digest(t):
    return hashlib.sha256(t.detach().contiguous().numpy().tobytes()).hexdigest()[:16]


def main():
    cfg = CONFIGS["c1"]
    t = make_inputs(cfg, seed=0)
    x = t["x"].clone().requires_grad_()
    p = t["p"].clone().requires_grad_()
    W1 = t["W1"].clone().requires_grad_()
    W2 = t["W2"].clone().requires_grad_()
    y = oracle.naive_expert_forward(x, p, t["experts"], W1, W2, torch.nn.GELU())
    dx, dp, dw1, dw2 = torch.autograd.grad(y, [x, p, W1, W2], t["dy"])
    eid, idx, off = oracle.route_ref(t["experts"], cfg.E)
    out = {
        "config": {"T": cfg.T, "d": cfg.d, "f": cfg.f, "E": cfg.E, "k": cfg.k, "activation": "gelu", "seed": 0},
        "inputs_sha256_16": {k: digest(v) for k, v in t.items()},
        "routing": {"sorted_expert_idxs": eid.tolist(), "sorted_scattered_idxs": idx.tolist(),
                    "expert_offsets": off.tolist()},
        "rows": [0, 17, 255],
        "Y_rows": y.detach()[[0, 17, 255], :8].tolist(),
        "dX_rows": dx[[0, 17, 255], :8].tolist(),
        "dg_rows": dp[[0, 17, 255]].tolist(),
        "sums": {"Y": float(y.double().sum()), "dX": float(dx.double().sum()), "dg": float(dp.double().sum()),
                 "dW1": float(dw1.double().sum()), "dW2": float(dw2.double().sum()),
                 "Y_abs": float(y.double().abs().sum()), "dW1_abs": float(dw1.double().abs().sum()),
                 "dW2_abs": float(dw2.double().abs().sum())},
    }
    with open(os.path.join(HERE, "c1_seed0.json"), "w") as fh:
        json.dump(out, fh)
    print("wrote c1_seed0.json")


if __name__ == "__main__":
    main()
