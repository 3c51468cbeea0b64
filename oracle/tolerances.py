"""Parity tolerances, stated once.

Elementwise bar for floating-point results (network outputs, activations, deltas, gradients,
encoding values):
    bf16: |a - b| <= 1e-3 + 1e-2 * |b|
    fp16: |a - b| <= 5e-4 + 5e-3 * |b|     (the absolute floor is the one of the reference's Python
                                            is_close, test/python/src/utils.py:9-33)
and the reference's own metric (include/common/result_check.h:83-102): max|a-b| / max(|a|_inf, |b|_inf).
Integer work (hash indices, cell selection, layout permutations) is bit-exact.

Where the bar is applied:
  * one layer at a time, GPU and oracle fed the SAME inputs: every element, no exception
    (the only difference left is the summation order inside the fp32 accumulator, at most one
    unit in the last place of T after rounding);
  * end to end through several layers: two correct evaluations that round to T after every layer
    diverge where an fp32 sum sits on a rounding boundary, and the flipped unit in the last place is
    then amplified by the following layers (the oracle's own T and double variants differ the same
    way, tests/test_oracle_mlp.py). There PROPAGATED = 2e-3 of the elements may leave the bar, none
    by more than 4x, and the reference's max-norm metric must hold at 1e-2 (bf16) / 5e-3 (fp16).
"""
import numpy as np

BF16, FP16, FP32 = 0, 1, 2
ELEMENTWISE = {BF16: (1e-3, 1e-2), FP16: (5e-4, 5e-3), FP32: (1e-6, 1e-5)}
MAX_NORM = {BF16: 1e-2, FP16: 5e-3, FP32: 1e-5}
PROPAGATED = 2e-3


def assert_close(a, b, dtype, what="", scale=1.0, frac_ok=0.0):
    """a: result, b: oracle. `scale` multiplies the absolute floor for quantities whose natural size is
    not O(1) (e.g. loss-scaled or batch-normalised gradients). `frac_ok` is the fraction of elements
    allowed outside the bar (0 unless stated at the call site)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    atol, rtol = ELEMENTWISE[dtype]
    bad = np.abs(a - b) > atol * scale + rtol * np.abs(b)
    n_bad = int(bad.sum())
    if frac_ok > 0:
        far = np.abs(a - b) > 4 * (atol * scale + rtol * np.abs(b))
        if far.any():
            i = np.unravel_index(np.argmax(far), a.shape)
            raise AssertionError(f"{what}: element {i} is beyond 4x the bar: got {a[i]!r}, oracle {b[i]!r}")
    if n_bad > frac_ok * a.size:
        i = np.unravel_index(np.argmax(np.abs(a - b) - rtol * np.abs(b)), a.shape)
        raise AssertionError(f"{what}: {n_bad}/{a.size} elements outside |a-b| <= {atol * scale:g} + {rtol:g}|b|; worst at {i}: "
                             f"got {a[i]!r}, oracle {b[i]!r}")


def bar_report(a, b, dtype, scale=1.0):
    """How a result stands against the strict elementwise bar: the number of elements outside it, that number as a fraction,
    and the worst ratio |a - b| / (atol * scale + rtol * |b|) (at most 1 when every element is inside)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    atol, rtol = ELEMENTWISE[dtype]
    ratio = np.abs(a - b) / (atol * scale + rtol * np.abs(b))
    n_out = int((ratio > 1.0).sum())
    return {"n": int(a.size), "n_outside": n_out, "frac_outside": n_out / max(int(a.size), 1), "worst_ratio": float(ratio.max()) if a.size else 0.0}


def max_norm_rel(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    d = max(np.abs(a).max(), np.abs(b).max())
    return np.abs(a - b).max() / d if d > 0 else np.abs(a - b).max()


def assert_propagated(a, b, dtype, what="", scale=1.0):
    """End-to-end bar for quantities that went through several rounded layers (see the module text)."""
    assert_close(a, b, dtype, what, scale=scale, frac_ok=PROPAGATED)
    r = max_norm_rel(a, b)
    assert r <= MAX_NORM[dtype], f"{what}: max-norm relative difference {r:g} > {MAX_NORM[dtype]:g}"
