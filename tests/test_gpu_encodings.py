"""Parity of the identity, frequency and spherical-harmonics kernels (through the C ABI) with the oracle.

fp32 outputs: |a - b| <= 2e-6 + 1e-5 |b| (sinf / cosf of the device against the host's, polynomial evaluation order);
half-precision outputs: the fp16 / bf16 bars of tests/tolerances.py.
"""
import json
import os

import numpy as np
import pytest
import torch

from tiny_dpcpp_nn import _lib
from tolerances import BF16, FP16, FP32, assert_close

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(__file__), "golden")


def close32(a, b, atol=2e-6, rtol=1e-5):
    assert np.all(np.abs(a - b) <= atol + rtol * np.abs(b)), float(np.abs(a - b).max())


@pytest.mark.parametrize("M,D,padded", [(1, 3, 3), (1000, 3, 16), (777, 5, 64), (4096, 1, 5346)])
def test_identity(tnn, oracle, M, D, padded):
    x = torch.rand((M, D), device=tnn.dev) * 4 - 2
    for scale, offset in ((1.0, 0.0), (2.5, -0.75)):
        out = tnn.identity_forward(x, scale, offset, padded)
        ref = oracle.identity_forward(x.cpu().numpy(), scale, offset, padded)
        assert np.array_equal(out.cpu().numpy(), ref)   # one multiply-add per element, rounded as on the host
    out16 = tnn.identity_forward(x, 1.0, 0.0, padded, FP16)
    assert_close(out16.float().cpu().numpy(), oracle.identity_forward(x.cpu().numpy(), 1.0, 0.0, padded), FP16, "identity fp16")


@pytest.mark.parametrize("M,D,n_freq,padded", [(1, 1, 1, 2), (1, 1, 1, 4), (2, 3, 2, 14), (5000, 3, 10, 64), (333, 2, 12, 48)])
def test_frequency_forward_and_backward(tnn, oracle, M, D, n_freq, padded):
    x = torch.rand((M, D), device=tnn.dev)
    out, dy = tnn.frequency_forward(x, n_freq, padded, want_dy_dx=True)
    ref, dy_ref = oracle.frequency_forward(x.cpu().numpy(), n_freq, padded, want_dy_dx=True)
    # sin / cos of arguments up to 2^11 pi: the device's and the host's float routines differ by a few ulps of the result
    close32(out.cpu().numpy(), ref, atol=2e-6)
    close32(dy.cpu().numpy(), dy_ref, atol=2e-6 * 2.0 ** n_freq * np.pi)
    width = D * n_freq * 2
    assert bool((out[:, width:] == 1).all())
    g = torch.randn((M, padded), device=tnn.dev)
    dx = tnn.frequency_backward(g, FP32, dy, D, n_freq)
    dx_ref = oracle.frequency_backward(g.cpu().numpy(), dy.cpu().numpy(), D, n_freq)
    close32(dx.cpu().numpy(), dx_ref, atol=1e-5 * float(np.abs(dx_ref).max()), rtol=1e-5)
    out_bf = tnn.frequency_forward(x, n_freq, padded, BF16)
    assert_close(out_bf.float().cpu().numpy(), ref, BF16, "frequency bf16")


def test_frequency_reference_vectors(tnn):
    """test/doctest_encodings.cpp:486-584 of the reference."""
    v = 1.234
    out = tnn.frequency_forward(torch.full((1, 1), v, device=tnn.dev), 1, 4).cpu().numpy()
    assert np.allclose(out, [[np.sin(np.pi * v), np.cos(np.pi * v), 1, 1]], atol=1e-4)


@pytest.mark.parametrize("degree", [1, 2, 3, 4, 5, 6, 7, 8])
def test_spherical_harmonics(tnn, oracle, degree):
    M, padded = 3001, ((degree * degree + 15) // 16) * 16
    x = torch.rand((M, 3), device=tnn.dev)
    out = tnn.sh_forward(x, degree, padded)
    ref = oracle.sh_forward(degree, x.cpu().numpy(), padded)
    close32(out.cpu().numpy(), ref, atol=2e-5, rtol=2e-5)   # float recurrences against the oracle's double ones
    assert bool((out[:, degree * degree:] == 1).all())
    out16 = tnn.sh_forward(x, degree, padded, FP16)
    assert_close(out16.float().cpu().numpy(), ref, FP16, "spherical harmonics fp16", scale=float(np.abs(ref).max()))


def test_spherical_harmonics_golden(tnn):
    fx = json.load(open(os.path.join(G, "spherical_harmonics_degree4.json")))
    x = torch.tensor([fx["input"]] * fx["n_rows"], device=tnn.dev)
    out = tnn.sh_forward(x, fx["degree"], 16).cpu().numpy()
    assert np.allclose(out, np.float32(fx["expected_row"])[None, :], atol=fx["atol"])
    # test/doctest_encodings.cpp:197-232
    out = tnn.sh_forward(torch.tensor([[0., 1., 2.], [3., 4., 5.]], device=tnn.dev), 1, 3).cpu().numpy()
    assert np.allclose(out, [[0.2821, 1.0, 1.0]] * 2, atol=1e-3)


def test_spherical_harmonics_all_64_polynomials(tnn):
    """The GPU kernel, bands 0-7, against the values of the reference's 64 polynomials (include/common/common_device.h:33-206)."""
    fx = json.load(open(os.path.join(G, "spherical_harmonics_degree8.json")))
    x = torch.tensor(fx["inputs"], dtype=torch.float32, device=tnn.dev)
    out = tnn.sh_forward(x, fx["degree"], 64).cpu().numpy()
    assert np.allclose(out, np.float64(fx["expected"]), atol=fx["atol"], rtol=1e-5)


def test_argument_checks(tnn):
    x = torch.zeros((8, 3), device=tnn.dev)
    o = torch.zeros((8, 64), device=tnn.dev)
    from gpu_harness import ptr
    L = tnn.lib
    assert L.tnn_identity_forward(ptr(x), 3, 1.0, 0.0, ptr(o), FP32, 2, 8, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert L.tnn_identity_forward(ptr(x), 0, 1.0, 0.0, ptr(o), FP32, 2, 8, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert L.tnn_frequency_forward(ptr(x), 3, 0, ptr(o), FP32, 64, None, 8, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert L.tnn_frequency_forward(ptr(x), 3, 4, ptr(o), FP32, 23, None, 8, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert L.tnn_frequency_backward(ptr(o), FP32, 64, ptr(o), 3, 4, ptr(x), 0, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert L.tnn_sh_forward(ptr(x), 9, ptr(o), FP32, 64, 8, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert L.tnn_sh_forward(ptr(x), 0, ptr(o), FP32, 64, 8, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert L.tnn_sh_forward(ptr(x), 4, ptr(o), FP32, 15, 8, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert L.tnn_sh_forward(ptr(x), 4, ptr(o), 7, 16, 8, None) == _lib.TNN_ERR_UNSUPPORTED
    assert L.tnn_identity_forward(None, 3, 1.0, 0.0, None, FP32, 3, 0, None) == _lib.TNN_OK   # an empty batch is fine
