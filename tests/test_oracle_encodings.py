"""Pins the oracle's identity, frequency and spherical-harmonics restatements against the data the reference's own
tests hold and against what the mathematics fixes (CPU only)."""
import json
import math
import os

import numpy as np

G = os.path.join(os.path.dirname(__file__), "golden")


def test_identity_closed_forms(oracle):
    # test/doctest_encodings.cpp:156-195: scale 1, offset 0 reproduces the input; test/python/test_encodings.py:593-608: padding
    x = np.full((2, 3), 1.23, np.float32)
    assert np.array_equal(oracle.identity_forward(x, 1.0, 0.0, 3), x)
    out = oracle.identity_forward(x, 2.0, -0.5, 8)
    assert np.allclose(out[:, :3], 1.23 * 2 - 0.5) and np.all(out[:, 3:] == 1.0)


def test_frequency_closed_forms(oracle):
    # test/doctest_encodings.cpp:486-584
    v = 1.234
    out = oracle.frequency_forward(np.float32([[v]]), 1, 2)
    assert np.allclose(out, [[math.sin(math.pi * v), math.cos(math.pi * v)]], atol=1e-4)
    out = oracle.frequency_forward(np.float32([[v]]), 1, 4)
    assert np.allclose(out, [[math.sin(math.pi * v), math.cos(math.pi * v), 1, 1]], atol=1e-4)
    x = np.float32([[0, 1, 2], [3, 4, 5]])
    out = oracle.frequency_forward(x, 2, 14)
    exp = []
    for row in x:
        for f in row:
            exp += [math.sin(math.pi * f), math.cos(math.pi * f), math.sin(2 * math.pi * f), math.cos(2 * math.pi * f)]
        exp += [1, 1]
    assert np.allclose(out.ravel(), exp, atol=1e-4)


def test_frequency_derivative_and_backward(oracle):
    rng = np.random.default_rng(0)
    x = rng.uniform(0, 1, (64, 3)).astype(np.float32)
    n_freq = 5
    out, dy = oracle.frequency_forward(x, n_freq, 32, want_dy_dx=True)
    # central differences in double on the closed form
    k = np.arange(3 * n_freq * 2)
    freq = (2.0 ** ((k // 2) % n_freq)) * math.pi
    feat = k // (2 * n_freq)
    arg = x.astype(np.float64)[:, feat] * freq + (k % 2) * math.pi / 2
    assert np.allclose(out[:, :30], np.sin(arg), atol=2e-5)
    assert np.allclose(dy, freq * np.cos(arg), rtol=1e-4, atol=2e-3)
    g = rng.standard_normal((64, 32)).astype(np.float32)
    dx = oracle.frequency_backward(g, dy, 3, n_freq)
    ref = (g[:, :30].astype(np.float64) * dy).reshape(64, 3, 2 * n_freq).sum(axis=2)
    assert np.allclose(dx, ref, rtol=1e-5, atol=1e-5)


def test_sh_golden_vectors(oracle):
    fx = json.load(open(os.path.join(G, "spherical_harmonics_degree4.json")))
    # the fixture's input passes through 2x - 1 inside the encoding: (1, 1, 1) stays (1, 1, 1)
    x = np.tile(np.float32(fx["input"]), (fx["n_rows"], 1))
    out = oracle.sh_forward(fx["degree"], x, 16)
    assert np.allclose(out, np.float32(fx["expected_row"])[None, :], atol=fx["atol"])
    # test/doctest_encodings.cpp:197-232: degree 1, padded to 3 columns with ones
    out = oracle.sh_forward(1, np.float32([[0, 1, 2], [3, 4, 5]]), 3)
    assert np.allclose(out, [[0.2821, 1.0, 1.0]] * 2, atol=1e-3)


def test_sh_recurrence_equals_the_references_expressions(oracle):
    """Bands 0-3 against the sixteen expressions the reference spells out; single members of bands 4-7 against the closed
    forms its comments give (include/common/common_device.h:74,88-89,103-104,113-115,133-135,150-152,178-180,201-203)."""
    rng = np.random.default_rng(1)
    pts = rng.uniform(0, 1, (200, 3)).astype(np.float32)   # not unit vectors: the expressions are polynomials
    out = oracle.sh_forward(8, pts, 64).astype(np.float64)
    d = (pts * np.float32(2) - np.float32(1)).astype(np.float64)
    sp = math.sqrt(math.pi)
    for i in range(len(pts)):
        x, y, z = d[i]
        assert np.allclose(out[i, :16], oracle.sh_explicit16(x, y, z), rtol=1e-6, atol=1e-6)
        x2, y2, z2 = x * x, y * y, z * z
        x4, y4, z4, x6, y6, z6 = x2 * x2, y2 * y2, z2 * z2, x2 ** 3, y2 ** 3, z2 ** 3
        spot = {
            16: 3 * math.sqrt(35) * x * y * (x2 - y2) / (4 * sp),
            24: 3 * math.sqrt(35) * (-6 * x2 * y2 + x4 + y4) / (16 * sp),
            30: math.sqrt(11) * z * (-70 * z2 + 63 * z4 + 15) / (16 * sp),
            35: 3 * math.sqrt(154) * x * (10 * x2 * y2 - x4 - 5 * y4) / (32 * sp),
            42: math.sqrt(13) * (105 * z2 - 315 * z4 + 231 * z6 - 5) / (32 * sp),
            48: math.sqrt(6006) * (15 * x2 * y4 - 15 * x4 * y2 + x6 - y6) / (64 * sp),
            56: math.sqrt(15) * z * (315 * z2 - 693 * z4 + 429 * z6 - 35) / (32 * sp),
            63: 3 * math.sqrt(715) * x * (-35 * x2 * y4 + 21 * x4 * y2 - x6 + 7 * y6) / (64 * sp),  # = 0.70716273 x (...)
        }
        for idx, val in spot.items():
            assert abs(out[i, idx] - val) <= 2e-6 * max(1.0, abs(val)), (idx, out[i, idx], val)


def test_sh_all_64_polynomials_of_the_reference(oracle):
    """Bands 0-7 against the values of the reference's 64 spelled-out polynomials (include/common/common_device.h:33-206) at
    seeded points, so that a slipped sign or normalisation in the higher bands fails here and not only at the user."""
    fx = json.load(open(os.path.join(G, "spherical_harmonics_degree8.json")))
    x = np.float32(fx["inputs"])
    out = oracle.sh_forward(fx["degree"], x, 64)
    ref = np.float64(fx["expected"])
    assert out.shape == ref.shape == (len(x), 64)
    assert np.allclose(out, ref, atol=fx["atol"], rtol=1e-5)
    # every band is present in the check: no column of the expected values is (near) constant zero
    assert (np.abs(ref).max(axis=0) > 1e-3).all()


def test_sh_orthonormal_on_the_sphere(oracle):
    """All 64 functions are orthonormal under the surface integral (Gauss-Legendre in cos(theta) x uniform in phi)."""
    n_t, n_p = 24, 48
    ct, wt = np.polynomial.legendre.leggauss(n_t)
    phi = (np.arange(n_p) + 0.5) * 2 * math.pi / n_p
    st = np.sqrt(1 - ct ** 2)
    d = np.stack([np.outer(st, np.cos(phi)).ravel(), np.outer(st, np.sin(phi)).ravel(), np.repeat(ct, n_p)], axis=1)
    w = np.repeat(wt, n_p) * (2 * math.pi / n_p)
    # the encoding maps its input through 2x - 1
    Y = oracle.sh_forward(8, ((d + 1) / 2).astype(np.float32), 64).astype(np.float64)
    gram = (Y * w[:, None]).T @ Y
    assert np.allclose(gram, np.eye(64), atol=2e-5)
