"""Cell order of a batch (tnn_grid_order_points) and the forward pass that reads it (tnn_grid_forward_ordered): the records are
a permutation of the rows with their own coordinates, sorted by coarse cell, and the encoded rows equal tnn_grid_forward's bit
for bit whatever the distribution of the points."""
import ctypes

import numpy as np
import pytest
import torch

from tolerances import FP16, FP32, assert_close

pytestmark = pytest.mark.gpu

CFG4 = dict(n_dims=2, n_levels=16, n_features_per_level=2, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.5)
CFG5 = dict(n_dims=3, n_levels=16, n_features_per_level=2, log2_hashmap_size=22, base_resolution=16, per_level_scale=1.447)


def points(kind, M, D, rng):
    if kind == "uniform":
        return rng.uniform(0, 1, (M, D)).astype(np.float32)
    if kind == "clustered":  # nearly everything in one coarse bin: the refinement's long-bin path
        x = (0.3 + 0.01 * rng.uniform(0, 1, (M, D))).astype(np.float32)
        x[::97] = rng.uniform(0, 1, (len(x[::97]), D))
        return x
    if kind == "identical":
        return np.full((M, D), 0.625, np.float32)
    x = rng.uniform(-0.5, 1.5, (M, D)).astype(np.float32)  # outside the unit cube, infinities and NaN among them
    x[3 % M], x[5 % M], x[7 % M] = np.nan, np.inf, -np.inf
    x[11 % M, 0] = np.nan
    return x


def records_of(tnn, d, xt):
    M = xt.shape[0]
    buf = tnn.grid_order(d, xt)
    torch.cuda.synchronize()
    rec = buf[: M * 16].view(torch.float32).reshape(M, 4).cpu().numpy()
    return buf, rec, rec[:, 3].copy().view(np.uint32)


@pytest.mark.parametrize("cfg", [CFG4, CFG5])
@pytest.mark.parametrize("kind", ["uniform", "clustered", "identical", "wild"])
@pytest.mark.parametrize("M", [1, 8, 1000, 4096 + 24, 300000])
def test_order_is_a_permutation_and_forward_is_unchanged(tnn, cfg, kind, M):
    D = cfg["n_dims"]
    rng = np.random.default_rng(M + D)
    x = points(kind, M, D, rng)
    xt = torch.from_numpy(x).to(tnn.dev)
    d = tnn.grid_desc(cfg, FP16)
    buf, rec, rows = records_of(tnn, d, xt)
    assert np.array_equal(np.sort(rows), np.arange(M, dtype=np.uint32)), "every row exactly once"
    assert np.array_equal(rec[:, :D].view(np.uint32), x[rows].view(np.uint32)), "a record carries its own row's coordinates"
    # sorted by the coarse key: the leading bits of every coordinate, first dimension fastest
    bits = 4 if D == 3 else 6
    with np.errstate(invalid="ignore", over="ignore"):
        s = x[rows].astype(np.float32) * np.float32(1 << bits)
        q = np.where(s > 0, np.minimum(np.where(np.isfinite(s), s, np.float32(1 << bits)), (1 << bits) - 1), 0).astype(np.int64)
    key = sum(q[:, k] << (bits * k) for k in range(D))
    assert np.all(np.diff(key) >= 0), "records are not in coarse-cell order"
    n = tnn.grid_n_params(d)
    table = torch.from_numpy(rng.uniform(-1, 1, n).astype(np.float32)).to(tnn.dev).to(torch.float16)
    if kind == "wild":
        xt = torch.nan_to_num(xt, nan=0.25, posinf=1.5, neginf=-0.5)  # the encoding of a NaN coordinate is not defined
        buf = tnn.grid_order(d, xt)
    plain = tnn.grid_forward(d, xt, table, 48, FP16)
    ordered = tnn.grid_forward_ordered(d, buf, table, 48, M, FP16)
    torch.cuda.synchronize()
    assert torch.equal(plain.view(torch.int16), ordered.view(torch.int16))


def test_ordered_forward_matches_the_oracle_and_every_variant(tnn, oracle):
    rng = np.random.default_rng(3)
    for cfg, pd, od in ((dict(CFG5, n_features_per_level=4, n_levels=8, interpolation="Smoothstep"), FP32, FP32),
                        (dict(CFG4, grid_type="Dense", n_levels=6, n_features_per_level=1), FP16, FP16),
                        (dict(CFG5, hash="Prime", n_features_per_level=8, n_levels=4, interpolation="Nearest"), FP16, FP32)):
        M = 20000
        x = rng.uniform(0, 1, (M, cfg["n_dims"])).astype(np.float32)
        d = tnn.grid_desc(cfg, pd)
        n = tnn.grid_n_params(d)
        table = oracle.round(rng.uniform(-1, 1, n), pd)
        tt = torch.from_numpy(table).to(tnn.dev).to(torch.float16 if pd == FP16 else torch.float32)
        xt = torch.from_numpy(x).to(tnn.dev)
        width = cfg["n_levels"] * cfg["n_features_per_level"]
        out = tnn.grid_forward_ordered(d, tnn.grid_order(d, xt), tt, width, M, od)
        ref = oracle.grid_forward(cfg, table, x, width)
        assert_close(out.to(torch.float32).cpu().numpy(), ref, od, f"ordered forward {cfg}")
        assert torch.equal(out.view(torch.uint8), tnn.grid_forward(d, xt, tt, width, od).view(torch.uint8))


def test_order_buffer_checks(tnn):
    from tiny_dpcpp_nn import _lib
    d = tnn.grid_desc(CFG5, FP16)
    x = torch.rand((64, 3), device=tnn.dev)
    need = tnn.lib.tnn_grid_order_bytes(ctypes.byref(d), 64)
    assert need >= 64 * 16
    buf = torch.empty(need + 256, dtype=torch.uint8, device=tnn.dev)
    p = buf.data_ptr()
    assert tnn.lib.tnn_grid_order_points(ctypes.byref(d), x.data_ptr(), 64, p, need - 1, None) == _lib.TNN_ERR_WORKSPACE
    assert tnn.lib.tnn_grid_order_points(ctypes.byref(d), x.data_ptr(), 64, p + 16, need, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert tnn.lib.tnn_grid_order_points(ctypes.byref(d), x.data_ptr(), 0, p, need, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert tnn.lib.tnn_grid_order_bytes(ctypes.byref(d), 0) == 0


def test_config_5_full_size_ordered(tnn, oracle):
    """BASELINE config 5's encoding at 2^21 points in cell order: equal to the plain pass bit for bit, a sample against the oracle."""
    M = 1 << 21
    d = tnn.grid_desc(CFG5, FP16)
    n = tnn.grid_n_params(d)
    gen = torch.Generator(device=tnn.dev).manual_seed(5)
    table = (torch.rand(n, device=tnn.dev, generator=gen) * 2e-4 - 1e-4).to(torch.float16)
    x = torch.rand((M, 3), device=tnn.dev, generator=gen)
    plain = tnn.grid_forward(d, x, table, 32, FP16)
    ordered = tnn.grid_forward_ordered(d, tnn.grid_order(d, x), table, 32, M, FP16)
    assert torch.equal(plain.view(torch.int16), ordered.view(torch.int16))
    rows = torch.randint(0, M, (4096,), device=tnn.dev, generator=gen)
    ref = oracle.grid_forward(CFG5, table.float().cpu().numpy(), x[rows].cpu().numpy(), 32)
    assert_close(ordered[rows].float().cpu().numpy(), ref, FP16, "config 5 ordered", scale=1e-4)


@pytest.mark.parametrize("cfg,pd", [(CFG4, FP16), (CFG5, FP16), (dict(CFG5, n_features_per_level=4, n_levels=8, interpolation="Smoothstep"), FP32),
                                    (dict(CFG4, grid_type="Dense", n_levels=6, n_features_per_level=1), FP16),
                                    (dict(CFG5, hash="Prime", n_features_per_level=8, n_levels=4, interpolation="Nearest"), FP16)])
@pytest.mark.parametrize("kind,M", [("uniform", 2011), ("uniform", 70000), ("clustered", 30001), ("identical", 777), ("uniform", 1),
                                    ("wild", 9001)])
def test_ordered_backward_matches_the_oracle(tnn, oracle, cfg, pd, kind, M):
    """tnn_grid_backward_ordered: the same contributions as tnn_grid_backward, summed per run of equal entries inside a wave
    first. fp32 sums in another order against the oracle's double sum: |err| <= 1e-5 x the largest entry (the bar of the
    plain call); identical points make runs of 16 in every wave and clustered ones runs of every length."""
    D, F, L = cfg["n_dims"], cfg["n_features_per_level"], cfg["n_levels"]
    rng = np.random.default_rng(M + 31 * D + F)
    x = points(kind, M, D, rng)
    if kind == "wild":  # points outside the unit cube: bins whose boxes do not fit (a NaN coordinate has no defined cell)
        x = np.nan_to_num(x, nan=0.25, posinf=1.5, neginf=-0.5)
    pw = L * F + 8
    d = tnn.grid_desc(cfg, pd)
    n = tnn.grid_n_params(d)
    xt = torch.from_numpy(x).to(tnn.dev)
    g = rng.standard_normal((M, pw)).astype(np.float32)
    gt = torch.from_numpy(g).to(tnn.dev)
    buf = tnn.grid_order(d, xt)
    grad = tnn.grid_backward_ordered(d, buf, gt, FP32).cpu().numpy()
    ref = oracle.grid_backward(cfg, x, g, n)
    bar = 1e-5 * max(1.0, np.abs(ref).max())
    assert np.abs(grad - ref).max() <= bar
    plain = tnn.grid_backward(d, xt, gt, FP32).cpu().numpy()
    assert np.abs(grad - plain).max() <= 2 * bar
    # accumulate mode adds on top of what the table holds
    twice = tnn.grid_backward_ordered(d, buf, gt, FP32, grad_t=torch.from_numpy(grad).to(tnn.dev), overwrite=False).cpu().numpy()
    assert np.abs(twice - 2 * ref).max() <= 2 * bar


def test_ordered_backward_config_4_full_size(tnn, oracle):
    cfg, M = CFG4, 1 << 18
    d = tnn.grid_desc(cfg, FP16)
    n = tnn.grid_n_params(d)
    gen = torch.Generator(device=tnn.dev).manual_seed(6)
    x = torch.rand((M, 2), device=tnn.dev, generator=gen)
    g = (torch.rand((M, 32), device=tnn.dev, generator=gen) - 0.5).to(torch.float16)
    grad = tnn.grid_backward_ordered(d, tnn.grid_order(d, x), g, FP16).cpu().numpy()
    ref = oracle.grid_backward(cfg, x.cpu().numpy(), g.to(torch.float32).cpu().numpy(), n)
    assert np.abs(grad - ref).max() <= 1e-5 * np.abs(ref).max() + 1e-4
    assert_close(grad, ref, FP32, "gradient table", scale=1e2, frac_ok=1e-4)


@pytest.mark.parametrize("cfg,M", [(CFG4, (1 << 20) + 8), (dict(CFG5, log2_hashmap_size=19), 1 << 20), (dict(CFG4, base_resolution=4, n_levels=12), 1 << 16)])
def test_ordered_backward_plans_at_other_sizes(tnn, cfg, M):
    """Batch sizes and level sets that change which levels take which route (stretch length, workgroups per coarse row, 3-D
    boxes): the ordered scatter against the plain one, both fp32 atomics: |a - b| <= 2e-5 x the largest entry."""
    d = tnn.grid_desc(cfg, FP16)
    gen = torch.Generator(device=tnn.dev).manual_seed(M % 1000)
    x = torch.rand((M, cfg["n_dims"]), device=tnn.dev, generator=gen)
    x[: M // 4] = x[: M // 4] * 0.05 + 0.4   # a quarter of the points in a small region: long coarse rows
    pw = cfg["n_levels"] * cfg["n_features_per_level"]
    g = (torch.rand((M, pw), device=tnn.dev, generator=gen) - 0.5).to(torch.float16)
    plain = tnn.grid_backward(d, x, g, FP16)
    ordered = tnn.grid_backward_ordered(d, tnn.grid_order(d, x), g, FP16)
    tnn.sync()
    scale = float(plain.abs().max())
    assert scale > 0
    assert float((plain - ordered).abs().max()) <= 2e-5 * scale
