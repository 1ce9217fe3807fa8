"""One place for the floating-point parity bars, so that every comparison is made - and reported - the same way.

Bars (elementwise, `err <= abs + rel * |want|`):
  float32             rel 1e-4, abs 1e-5
  bfloat16 / float16  rel 2e-2, abs 1e-2

The absolute term is meant for values of magnitude about one.  Rule used everywhere: when the reference tensor's
largest magnitude `m` exceeds 1, the absolute term is multiplied by `m` (a sum of n products of 16-bit values
carries a rounding error that grows with its own magnitude); when `m <= 1` the literal, unscaled bar is asserted.
`check` also records the observed errors; at the end of the session they are written, as a table of max |err|,
max |err| / m and the share of the bar that was used, to the file the environment variable
SCATTERMOE_PARITY_REPORT names (no report when it is unset).
"""
import os

import torch

BARS = {torch.float32: (1e-4, 1e-5), torch.bfloat16: (2e-2, 1e-2), torch.float16: (2e-2, 1e-2)}

REPORT = []          # (name, dtype, m, max abs err, max err / m, worst err / bound, kind, share outside literal bar, rel. Frobenius)

ULP_BITS = {torch.float32: 23, torch.bfloat16: 7, torch.float16: 10}


def ulp(m, dtype):
    """Spacing of `dtype` values at magnitude m."""
    import math
    return 2.0 ** (math.floor(math.log2(m)) - ULP_BITS[dtype]) if m > 0 else 0.0


def check(name, got, want, dtype, record=True, literal=False):
    """Assert `got` (any device / dtype) against the float reference `want` at the bar of `dtype`.

    `literal`: for a reference that was itself rounded to the storage type wherever the path stores a tensor
    (oracle.rounded_glu_*), so that what is left to differ is the order of the float32 sums.  A different order
    flips the rounding of a stored intermediate now and then (by one unit in ITS last place), and such a flip
    reaches the results that intermediate feeds at its own size, however small they are.  Asserted therefore:
    at least 99.5 % of the elements (all but two of a small sample) inside the literal bar (abs + rel * |want|,
    nothing scaled); every element inside
    the literal bar plus one unit in the last place of the tensor's largest magnitude; relative Frobenius error
    below 1e-3 (a tenth of what the format's own rounding leaves against an unrounded reference)."""
    rel, ab = BARS[dtype]
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    assert got.shape == want.shape, "%s: shape %s vs %s" % (name, tuple(got.shape), tuple(want.shape))
    if want.numel() == 0:
        return 0.0
    assert bool(torch.isfinite(got).all()), "%s: non-finite values" % name
    m = float(want.abs().max())
    scale = m if m > 1.0 and not literal else 1.0
    err = (got - want).abs()
    lit = ab + rel * want.abs()
    bound = lit + ulp(m, dtype) if literal else ab * scale + rel * want.abs()
    used = float((err / bound).max())
    outside = float((err > lit).float().mean())
    frob = float(err.norm() / want.norm().clamp_min(1e-30))
    kind = "literal + 1 ulp of max" if literal else ("scaled x%.3g" % scale if scale > 1.0 else "literal")
    if record:
        REPORT.append((name, str(dtype).replace("torch.", ""), m, float(err.max()), float(err.max()) / max(m, 1e-30),
                       used, kind, outside, frob))
    assert used <= 1.0, "%s: max err %.4g (|ref| max %.4g), %.2f of the %s bar" % (name, float(err.max()), m, used, kind)
    if literal:
        n_out = int((err > lit).sum())
        assert n_out <= max(2, 0.005 * err.numel()), "%s: %d of %d elements outside the literal bar" % (name, n_out, err.numel())
        assert frob <= 1e-3, "%s: relative Frobenius error %.3g" % (name, frob)
    return used


def write_report(path):
    if not REPORT:
        return
    lines = ["| tensor | dtype | max abs(ref) | max abs err | err / max abs(ref) | share of bar used | bar | "
             "outside the literal bar | rel. Frobenius err |",
             "|---|---|---|---|---|---|---|---|---|"]
    for name, dt, m, e, r, u, kind, outside, frob in REPORT:
        lines.append("| %s | %s | %.4g | %.3g | %.3g | %.2f | %s | %.3f %% | %.2g |" % (name, dt, m, e, r, u, kind, 100 * outside, frob))
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def maybe_write_report():
    path = os.environ.get("SCATTERMOE_PARITY_REPORT")
    if REPORT and path:
        write_report(path)
