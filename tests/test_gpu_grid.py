"""Parity of the hash-grid kernels (through the C ABI) with the oracle: indices bit-exact,
values within the stated tolerance."""
import ctypes
import json
import os

import numpy as np
import pytest
import torch

from tolerances import BF16, FP16, FP32, assert_close, max_norm_rel

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(__file__), "golden")

CFG4 = dict(n_dims=2, n_levels=16, n_features_per_level=2, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.5)
CFG5 = dict(n_dims=3, n_levels=16, n_features_per_level=2, log2_hashmap_size=22, base_resolution=16, per_level_scale=1.447)


def test_desc_matches_oracle_tables(tnn, oracle):
    for cfg in (CFG4, CFG5, dict(CFG5, per_level_scale=2.0, log2_hashmap_size=19)):
        d = tnn.grid_desc(cfg)
        off, sc, res = oracle.grid_offsets(cfg["n_dims"], cfg["n_levels"], cfg["log2_hashmap_size"], cfg["base_resolution"], cfg["per_level_scale"])
        assert list(d.offsets[:17]) == off.tolist()
        assert np.array_equal(np.array(d.scales[:16], np.float32), sc)
        assert list(d.resolutions[:16]) == res.tolist()
        assert tnn.grid_n_params(d) == int(off[-1]) * 2


def test_golden_vector(tnn):
    # test/doctest_encodings.cpp:234-285, fp32 table as in the reference
    g = json.load(open(os.path.join(G, "grid_forward_3d.json")))
    cfg = dict(n_dims=3, n_levels=16, n_features_per_level=2, log2_hashmap_size=19, base_resolution=16, per_level_scale=2.0)
    d = tnn.grid_desc(cfg)
    n = tnn.grid_n_params(d)
    table = torch.from_numpy((np.arange(n, dtype=np.float64) / (n / 2.0) - 1.0).astype(np.float32)).to(tnn.dev)
    x = torch.ones((1, 3), device=tnn.dev)
    out = tnn.grid_forward(d, x, table, 32).cpu().numpy()[0]
    assert max_norm_rel(out, np.array(g["expected"])) <= g["tolerance"]
    # zero dL/dy: gradient table overwritten with zeros, parameters untouched (:286-341)
    grad = tnn.grid_backward(d, x, torch.zeros((1, 32), device=tnn.dev), FP32)
    assert float(grad.abs().max()) == 0.0


@pytest.mark.parametrize("cfg", [CFG4, CFG5, dict(CFG4, hash="Prime"), dict(CFG5, hash="ReversedPrime"),
                                 dict(CFG4, grid_type="Dense", n_levels=6), dict(CFG5, grid_type="Tiled"),
                                 dict(CFG5, n_levels=4, log2_hashmap_size=10)])
def test_indices_bit_exact(tnn, oracle, cfg):
    rng = np.random.default_rng(11)
    x = rng.uniform(0, 1, (4096, cfg["n_dims"])).astype(np.float32)
    x[:8] = np.array([0.0, 1.0, 0.5, 0.25, 0.999999, 1e-7, 0.75, 0.333333343], np.float32)[:, None]
    d = tnn.grid_desc(cfg)
    got = tnn.grid_indices(d, torch.from_numpy(x).to(tnn.dev))
    assert np.array_equal(got, oracle.grid_indices(cfg, x))


@pytest.mark.parametrize("cfg", [CFG4, CFG5])
@pytest.mark.parametrize("param_dtype,out_dtype", [(FP32, FP32), (FP16, FP16), (FP16, BF16), (FP16, FP32)])
def test_forward_values(tnn, oracle, cfg, param_dtype, out_dtype):
    rng = np.random.default_rng(12)
    M = 3000
    x = rng.uniform(0, 1, (M, cfg["n_dims"])).astype(np.float32)
    d = tnn.grid_desc(cfg, param_dtype)
    n = tnn.grid_n_params(d)
    table = rng.uniform(-1, 1, n).astype(np.float32)
    if param_dtype == FP16:
        table = oracle.round(table, FP16)
    tt = torch.from_numpy(table).to(tnn.dev).to(torch.float16 if param_dtype == FP16 else torch.float32)
    out = tnn.grid_forward(d, torch.from_numpy(x).to(tnn.dev), tt, 64, out_dtype).to(torch.float32).cpu().numpy()
    ref = oracle.grid_forward(cfg, table, x, 64)
    if out_dtype == FP32:
        # same corner order, same fused multiply-add: identical up to the last bit of the fp32 blend
        assert np.abs(out - ref).max() <= 1e-6
    else:
        assert np.array_equal(out, oracle.round(ref, out_dtype)) or np.abs(out - ref).max() <= 2 ** -8
        assert_close(out, ref, out_dtype, "encoded values")
    assert np.all(out[:, 32:] == 0)


@pytest.mark.parametrize("cfg", [CFG4, CFG5, dict(CFG4, interpolation="Smoothstep"), dict(CFG4, interpolation="Nearest"),
                                 dict(CFG5, n_features_per_level=4, n_levels=8), dict(CFG4, n_features_per_level=1), dict(CFG4, n_features_per_level=8, n_levels=4),
                                 dict(CFG4, grid_type="Dense", n_levels=7), dict(CFG5, grid_type="Tiled", n_levels=6, log2_hashmap_size=15),
                                 dict(CFG5, hash="Prime", log2_hashmap_size=14, n_features_per_level=1)])
def test_forward_backward_variants(tnn, oracle, cfg):
    rng = np.random.default_rng(13)
    M = 2011  # no multiple of the (point, level) pairs a workgroup of the backward takes, whatever the feature count
    F, L = cfg["n_features_per_level"], cfg["n_levels"]
    pw = L * F + 8
    x = rng.uniform(0, 1, (M, cfg["n_dims"])).astype(np.float32)
    d = tnn.grid_desc(cfg)
    n = tnn.grid_n_params(d)
    table = rng.uniform(-1, 1, n).astype(np.float32)
    xt = torch.from_numpy(x).to(tnn.dev)
    out = tnn.grid_forward(d, xt, torch.from_numpy(table).to(tnn.dev), pw).cpu().numpy()
    assert np.abs(out - oracle.grid_forward(cfg, table, x, pw)).max() <= 1e-6
    g = rng.standard_normal((M, pw)).astype(np.float32)
    grad = tnn.grid_backward(d, xt, torch.from_numpy(g).to(tnn.dev), FP32).cpu().numpy()
    ref = oracle.grid_backward(cfg, x, g, n)
    # fp32 atomics in arbitrary order against a double sum: |err| <= few ulp * sum of |terms|
    assert np.abs(grad - ref).max() <= 1e-5 * max(1.0, np.abs(ref).max())
    # accumulate mode adds on top
    grad2 = tnn.grid_backward(d, xt, torch.from_numpy(g).to(tnn.dev), FP32, grad_t=torch.from_numpy(grad).to(tnn.dev), overwrite=False).cpu().numpy()
    assert np.abs(grad2 - 2 * ref).max() <= 2e-5 * max(1.0, np.abs(ref).max())


def test_backward_half_precision_dy(tnn, oracle):
    cfg = CFG4
    rng = np.random.default_rng(14)
    M = 4096
    x = rng.uniform(0, 1, (M, 2)).astype(np.float32)
    d = tnn.grid_desc(cfg, FP16)
    n = tnn.grid_n_params(d)
    for dt, tdt in ((BF16, torch.bfloat16), (FP16, torch.float16)):
        g = oracle.round(rng.standard_normal((M, 64)), dt)
        grad = tnn.grid_backward(d, torch.from_numpy(x).to(tnn.dev), torch.from_numpy(g).to(tnn.dev).to(tdt), dt).cpu().numpy()
        ref = oracle.grid_backward(cfg, x, g, n)
        assert np.abs(grad - ref).max() <= 1e-5 * max(1.0, np.abs(ref).max())


def test_argument_checks(tnn):
    from tiny_dpcpp_nn import _lib
    d = _lib.GridDesc()
    rc = tnn.lib.tnn_grid_desc_init(ctypes.byref(d), 3, 129, 2, 19, 16, 2.0, 0, 1, 1, FP32)
    assert rc == _lib.TNN_ERR_INVALID_ARGUMENT  # include/encodings/grid.h:607-610
    rc = tnn.lib.tnn_grid_desc_init(ctypes.byref(d), 3, 16, 3, 19, 16, 2.0, 0, 1, 1, FP32)
    assert rc == _lib.TNN_ERR_INVALID_ARGUMENT  # include/encodings/grid.h:1067-1090
    d = tnn.grid_desc(CFG5)
    x = torch.zeros((8, 3), device=tnn.dev)
    out = torch.zeros((8, 32), device=tnn.dev)
    tab = torch.zeros(16, device=tnn.dev)
    from gpu_harness import ptr
    assert tnn.lib.tnn_grid_forward(ctypes.byref(d), ptr(x), ptr(tab), ptr(out), FP32, 16, 8, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert tnn.lib.tnn_grid_forward(ctypes.byref(d), ptr(x), ptr(tab), ptr(out), FP32, 0, 8, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert tnn.lib.tnn_grid_backward(ctypes.byref(d), ptr(x), ptr(out), FP32, 32, ptr(tab), 1, 0, None) == _lib.TNN_ERR_INVALID_ARGUMENT


def test_baseline_config_5_full_size(tnn, oracle):
    """BASELINE config 5 encoding: 3-D, 2^21 points, log2 22, fp16 table U(+-1e-4); indices of a seeded
    sample bit-exact, values compared on the full batch."""
    cfg = CFG5
    M = 1 << 21
    d = tnn.grid_desc(cfg, FP16)
    n = tnn.grid_n_params(d)
    assert n == 85038528
    gen = torch.Generator(device=tnn.dev).manual_seed(5)
    table = (torch.rand(n, device=tnn.dev, generator=gen) * 2e-4 - 1e-4).to(torch.float16)
    x = torch.rand((M, 3), device=tnn.dev, generator=gen)
    out = tnn.grid_forward(d, x, table, 32, FP16)
    xs = x.cpu().numpy()
    ref = oracle.grid_forward(cfg, table.to(torch.float32).cpu().numpy(), xs, 32)
    o = out.to(torch.float32).cpu().numpy()
    # values are O(1e-4): the absolute floor of the fp16 bar is scaled to that magnitude
    assert_close(o, ref, FP16, "config 5 encoding", scale=1e-4)
    assert max_norm_rel(o, ref) < 5e-3
    sub = slice(0, 1 << 16)
    assert np.array_equal(tnn.grid_indices(d, x[sub].contiguous()), oracle.grid_indices(cfg, xs[sub]))
    # size-independent property: the weights of a point sum to 1, so a constant table encodes to the constant
    const = torch.full((n,), 0.5, dtype=torch.float16, device=tnn.dev)
    oc = tnn.grid_forward(d, x, const, 32, FP32)
    assert float((oc - 0.5).abs().max()) <= 1e-6


def test_baseline_config_4_backward_full_size(tnn, oracle):
    """BASELINE config 4 encoding backward: 2-D, 2^18 points, gradient table against the oracle, and the
    adjoint identity <fwd(table), g> == <table, bwd(g)>."""
    cfg = CFG4
    M = 1 << 18
    d = tnn.grid_desc(cfg, FP16)
    n = tnn.grid_n_params(d)
    assert n == 7658384
    gen = torch.Generator(device=tnn.dev).manual_seed(6)
    x = torch.rand((M, 2), device=tnn.dev, generator=gen)
    g = (torch.rand((M, 32), device=tnn.dev, generator=gen) - 0.5).to(torch.float16)
    grad = tnn.grid_backward(d, x, g, FP16)
    ref = oracle.grid_backward(cfg, x.cpu().numpy(), g.to(torch.float32).cpu().numpy(), n)
    gh = grad.cpu().numpy()
    assert np.abs(gh - ref).max() <= 1e-5 * np.abs(ref).max() + 1e-4
    assert_close(gh, ref, FP32, "gradient table", scale=1e2, frac_ok=1e-4)
    table = (torch.rand(n, device=tnn.dev, generator=gen) - 0.5).to(torch.float16)
    out = tnn.grid_forward(d, x, table, 32, FP32)
    lhs = float((out.double() * g.double()).sum())
    rhs = float((table.double() * grad.double()).sum())
    # both sides are sums of 8M signed terms; the fp32 atomics round each gradient entry, so the bar is
    # relative to the sum of magnitudes
    mag = float((out.double().abs() * g.double().abs()).sum())
    assert abs(lhs - rhs) <= 1e-6 * mag


@pytest.mark.parametrize("cfg,M", [(CFG4, 1 << 16), (CFG5, 1 << 15), (dict(CFG4, n_features_per_level=4, n_levels=8), 5000)])
def test_backward_packed_fp16_table(tnn, oracle, cfg, M):
    """tnn_grid_backward_packed: same scatter, fp16 table, one packed atomic per pair of features. Every addition rounds to
    fp16, so an entry that receives n contributions is within about sqrt(n) * 2^-11 of the fp32 sum: 2e-2 of the largest
    entry per element, 2e-3 in the Frobenius norm. Overwrite zeroes the table first, Accumulate adds to it."""
    from gpu_harness import ptr
    from tiny_dpcpp_nn import _lib
    d = tnn.grid_desc(cfg, FP16)
    n = tnn.grid_n_params(d)
    D = cfg["n_dims"]
    pw = cfg["n_levels"] * cfg["n_features_per_level"]
    gen = torch.Generator(device=tnn.dev).manual_seed(8)
    x = torch.rand((M, D), device=tnn.dev, generator=gen)
    g = (torch.rand((M, pw), device=tnn.dev, generator=gen) - 0.5).to(torch.float16)
    table = torch.full((n,), 7.0, dtype=torch.float16, device=tnn.dev)
    _lib.check(tnn.lib.tnn_grid_backward_packed(ctypes.byref(d), ptr(x), ptr(g), FP16, pw, ptr(table), 1, M, tnn.stream()))
    ref = oracle.grid_backward(cfg, x.cpu().numpy(), g.float().cpu().numpy(), n)
    got = table.float().cpu().numpy()
    top = np.abs(ref).max()
    assert np.abs(got - ref).max() <= 2e-2 * top
    assert np.linalg.norm(got - ref) <= 2e-3 * np.linalg.norm(ref)
    _lib.check(tnn.lib.tnn_grid_backward_packed(ctypes.byref(d), ptr(x), ptr(g), FP16, pw, ptr(table), 0, M, tnn.stream()))
    assert np.linalg.norm(table.float().cpu().numpy() - 2 * ref) <= 4e-3 * np.linalg.norm(ref)
    odd = tnn.grid_desc(dict(cfg, n_features_per_level=1), FP16)
    assert tnn.lib.tnn_grid_backward_packed(ctypes.byref(odd), ptr(x), ptr(g), FP16, pw, ptr(table), 1, 8, tnn.stream()) == _lib.TNN_ERR_UNSUPPORTED
