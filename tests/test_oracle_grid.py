"""Pins the oracle's hash-grid functions: the reference's golden vector, its zero-gradient case,
the level table the constructor must produce, brute-force dense indexing, and invariants."""
import json
import os

import numpy as np
import pytest

G = os.path.join(os.path.dirname(__file__), "golden")

CFG4 = dict(n_dims=2, n_levels=16, n_features_per_level=2, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.5)
CFG5 = dict(n_dims=3, n_levels=16, n_features_per_level=2, log2_hashmap_size=22, base_resolution=16, per_level_scale=1.447)


def golden_cfg():
    d = json.load(open(os.path.join(G, "grid_forward_3d.json")))
    cfg = dict(n_dims=d["n_dims"], n_levels=d["n_levels"], n_features_per_level=d["n_features_per_level"],
               log2_hashmap_size=d["log2_hashmap_size"], base_resolution=d["base_resolution"],
               per_level_scale=d["per_level_scale"], grid_type=d["grid_type"], hash=d["hash"], interpolation=d["interpolation"])
    return d, cfg


def test_forward_golden_vector(oracle):
    # test/doctest_encodings.cpp:234-285
    d, cfg = golden_cfg()
    off, _, _ = oracle.grid_offsets(cfg["n_dims"], cfg["n_levels"], cfg["log2_hashmap_size"], cfg["base_resolution"], cfg["per_level_scale"])
    n = int(off[-1]) * cfg["n_features_per_level"]
    table = (np.arange(n, dtype=np.float64) / (n / 2.0) - 1.0).astype(np.float32)
    out = oracle.grid_forward(cfg, table, np.array([d["input"]], np.float32), d["padded_output_width"])[0]
    exp = np.array(d["expected"])
    assert np.abs(out - exp).max() / max(np.abs(out).max(), np.abs(exp).max()) <= d["tolerance"]


def test_backward_zero_gradient_case(oracle):
    # test/doctest_encodings.cpp:286-341: zero dL/dy overwrites a 0.123-filled gradient table with zeros
    _, cfg = golden_cfg()
    off, _, _ = oracle.grid_offsets(3, 16, 19, 16, 2.0)
    n = int(off[-1]) * 2
    grad = oracle.grid_backward(cfg, np.ones((1, 3), np.float32), np.zeros((1, 32), np.float32), n)
    assert np.all(grad == 0)


def test_level_tables_of_the_baseline_configs(oracle):
    # closed form of include/encodings/grid.h:613-644
    off, sc, res = oracle.grid_offsets(2, 16, 19, 16, 1.5)
    sizes = np.diff(off.astype(np.int64))
    assert sizes[0] == 256 and sizes[9] == 379456 and np.all(sizes[10:] == 524288)
    assert int(off[-1]) == 3829192
    for l in range(16):
        s = np.float32(np.exp2(np.float32(l) * np.log2(np.float32(1.5)))) * np.float32(16) - np.float32(1)
        assert abs(sc[l] - s) <= 4 * np.spacing(np.float32(s))
        assert res[l] == int(np.ceil(sc[l])) + 1
        dense = -(-(int(res[l]) ** 2) // 8) * 8
        assert sizes[l] == min(dense, 1 << 19)
    off, sc, res = oracle.grid_offsets(3, 16, 22, 16, 1.447)
    sizes = np.diff(off.astype(np.int64))
    assert sizes[0] == 4096 and sizes[6] == 3176528 and np.all(sizes[7:] == 4194304)
    assert int(off[-1]) == 42519264


@pytest.mark.parametrize("n_dims", [2, 3])
def test_dense_levels_index_is_row_major_brute_force(oracle, n_dims):
    cfg = dict(n_dims=n_dims, n_levels=4, n_features_per_level=2, log2_hashmap_size=24, base_resolution=4, per_level_scale=2.0)
    rng = np.random.default_rng(0)
    x = rng.uniform(0, 1, (200, n_dims)).astype(np.float32)
    idx, cells = oracle.grid_indices(cfg, x, want_cells=True)
    off, sc, res = oracle.grid_offsets(n_dims, 4, 24, 4, 2.0)
    for l in range(4):
        size = int(off[l + 1] - off[l])
        assert size >= int(res[l]) ** n_dims  # dense
        pos = np.float32(sc[l]) * x + np.float32(0.5)
        assert np.array_equal(cells[:, l, :], np.floor(pos).astype(np.uint32))
        for c in range(1 << n_dims):
            loc = cells[:, l, :].astype(np.int64) + np.array([(c >> d) & 1 for d in range(n_dims)])
            lin = sum(loc[:, d] * int(res[l]) ** d for d in range(n_dims)) % size
            assert np.array_equal(idx[:, l, c], lin.astype(np.uint32))


def test_hashed_levels_use_the_xor_prime_hash(oracle):
    primes = [1, 2654435761, 805459861]
    x = np.random.default_rng(1).uniform(0, 1, (100, 3)).astype(np.float32)
    idx, cells = oracle.grid_indices(CFG5, x, want_cells=True)
    off, sc, res = oracle.grid_offsets(3, 16, 22, 16, 1.447)
    l = 12
    assert off[l + 1] - off[l] == 1 << 22
    for c in range(8):
        loc = cells[:, l, :].astype(np.uint64) + np.array([(c >> d) & 1 for d in range(3)], np.uint64)
        h = np.zeros(100, np.uint64)
        for d in range(3):
            h ^= (loc[:, d] * np.uint64(primes[d])) & np.uint64(0xFFFFFFFF)
        assert np.array_equal(idx[:, l, c], (h % np.uint64(1 << 22)).astype(np.uint32))


def test_wraparound_at_upper_boundary(oracle):
    # x = 1.0 puts cell+1 == resolution on dense levels: the index wraps with % size as in common_device.h:764
    cfg = dict(n_dims=2, n_levels=2, n_features_per_level=2, log2_hashmap_size=19, base_resolution=16, per_level_scale=2.0)
    idx, cells = oracle.grid_indices(cfg, np.ones((1, 2), np.float32), want_cells=True)
    off, sc, res = oracle.grid_offsets(2, 2, 19, 16, 2.0)
    assert cells[0, 0, 0] == 15 and res[0] == 16
    assert idx[0, 0, 3] == (16 + 16 * 16) % 256


@pytest.mark.parametrize("cfg", [CFG4, CFG5])
def test_constant_table_gives_constant_output_and_adjoint_identity(oracle, cfg):
    off, _, _ = oracle.grid_offsets(cfg["n_dims"], 16, cfg["log2_hashmap_size"], 16, cfg["per_level_scale"])
    n = int(off[-1]) * 2
    rng = np.random.default_rng(2)
    x = rng.uniform(0, 1, (64, cfg["n_dims"])).astype(np.float32)
    out = oracle.grid_forward(cfg, np.full(n, 0.75, np.float32), x, 40)
    assert np.allclose(out[:, :32], 0.75, atol=1e-6) and np.all(out[:, 32:] == 0)
    # <fwd(table), g> == <table, bwd(g)> : the forward is linear in the table
    table = rng.standard_normal(n).astype(np.float32)
    g = rng.standard_normal((64, 40)).astype(np.float32)
    lhs = float((oracle.grid_forward(cfg, table, x, 40).astype(np.float64) * g).sum())
    grad = oracle.grid_backward(cfg, x, g, n)
    rhs = float((table.astype(np.float64) * grad).sum())
    assert abs(lhs - rhs) < 1e-4 * max(1.0, abs(lhs))
    # per level, the gradients of feature f sum to sum_i dL/dy[i, l*F+f] (the weights sum to 1)
    for l in (0, 5, 15):
        gl = grad[int(off[l]) * 2:int(off[l + 1]) * 2].reshape(-1, 2).astype(np.float64).sum(0)
        assert np.allclose(gl, g[:, 2 * l:2 * l + 2].astype(np.float64).sum(0), atol=1e-4)


def test_nearest_and_smoothstep(oracle):
    cfg = dict(CFG4, interpolation="Nearest")
    off, _, _ = oracle.grid_offsets(2, 16, 19, 16, 1.5)
    n = int(off[-1]) * 2
    table = np.arange(n, dtype=np.float32)
    x = np.array([[0.3, 0.6]], np.float32)
    out = oracle.grid_forward(cfg, table, x, 32)
    idx = oracle.grid_indices(cfg, x)
    for l in range(16):
        assert out[0, 2 * l] == table[(int(off[l]) + int(idx[0, l, 0])) * 2]
    # smoothstep keeps the partition of unity
    out = oracle.grid_forward(dict(CFG4, interpolation="Smoothstep"), np.full(n, 2.0, np.float32), x, 32)
    assert np.allclose(out, 2.0, atol=1e-6)
