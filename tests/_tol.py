"""One place for the floating-point parity bars, so that every comparison is made - and reported - the same way.

Bars (elementwise, `err <= abs + rel * |want|`):
  float32             rel 1e-4, abs 1e-5
  bfloat16 / float16  rel 2e-2, abs 1e-2

The absolute term is meant for values of magnitude about one.  Rule used everywhere: when the reference tensor's
largest magnitude `m` exceeds 1, the absolute term is multiplied by `m` (a sum of n products of 16-bit values
carries a rounding error that grows with its own magnitude); when `m <= 1` the literal, unscaled bar is asserted.
`check` also records the observed errors; the session writes them to `gpurun_out/parity_errors.md` (a table of
max |err|, max |err| / m and the share of the bar that was used) when that folder exists.
"""
import os

import torch

BARS = {torch.float32: (1e-4, 1e-5), torch.bfloat16: (2e-2, 1e-2), torch.float16: (2e-2, 1e-2)}

REPORT = []          # (name, dtype, m, max abs err, max err / m, worst err / bound, "literal" | "scaled")


def check(name, got, want, dtype, record=True):
    """Assert `got` (any device / dtype) against the float reference `want` at the bar of `dtype`."""
    rel, ab = BARS[dtype]
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    assert got.shape == want.shape, "%s: shape %s vs %s" % (name, tuple(got.shape), tuple(want.shape))
    if want.numel() == 0:
        return 0.0
    assert bool(torch.isfinite(got).all()), "%s: non-finite values" % name
    m = float(want.abs().max())
    scale = m if m > 1.0 else 1.0
    err = (got - want).abs()
    bound = ab * scale + rel * want.abs()
    used = float((err / bound).max())
    if record:
        REPORT.append((name, str(dtype).replace("torch.", ""), m, float(err.max()), float(err.max()) / max(m, 1e-30),
                       used, "scaled x%.3g" % scale if scale > 1.0 else "literal"))
    assert used <= 1.0, "%s: max err %.4g (|ref| max %.4g), %.2f of the %s bar" % (
        name, float(err.max()), m, used, "scaled" if scale > 1.0 else "literal")
    return used


def write_report(path):
    if not REPORT:
        return
    lines = ["| tensor | dtype | max abs(ref) | max abs err | err / max abs(ref) | share of bar used | bar |",
             "|---|---|---|---|---|---|---|"]
    for name, dt, m, e, r, u, kind in REPORT:
        lines.append("| %s | %s | %.4g | %.3g | %.3g | %.2f | %s |" % (name, dt, m, e, r, u, kind))
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def maybe_write_report():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = os.path.join(root, "gpurun_out")
    if REPORT and os.path.isdir(out):
        write_report(os.path.join(out, "parity_errors.md"))
