"""Pins the oracle's weight-layout functions against the reference's own golden vectors."""
import json
import os

import numpy as np

G = os.path.join(os.path.dirname(__file__), "golden")


def test_get_packed_weights_golden(oracle):
    # test/doctest_packing.cpp:21-46
    d = json.load(open(os.path.join(G, "packing_16x16x2.json")))
    unpacked = np.arange(1, 513, dtype=np.float32)
    packed = oracle.pack_weights(unpacked, 2, 16)
    assert packed.astype(int).tolist() == d["packed"]


def test_packed_coord_point_values(oracle):
    # test/doctest_common.cpp:25-119
    d = json.load(open(os.path.join(G, "packed_coords.json")))
    for idx, rows, cols, exp in d["to_packed"]:
        assert oracle.to_packed(idx, rows, cols) == exp
    for idx, rows, cols, exp in d["from_packed"]:
        assert oracle.from_packed(idx, rows, cols) == exp


def test_pack_4x4_golden(oracle):
    # test/python/test_packing.py:9-48 ; the C entry point is square-matrix only, so go through the coordinate map
    d = json.load(open(os.path.join(G, "packed_coords.json")))["pack_4x4"]
    A = np.array(d["unpacked"]).ravel()
    P = np.zeros(16, int)
    for idx in range(16):
        P[oracle.to_packed(idx, 4, 4)] = A[idx]
    assert P.reshape(4, 4).tolist() == d["packed"]
    U = np.array([P[oracle.to_packed(i, 4, 4)] for i in range(16)])
    assert U.tolist() == A.tolist()


def test_pack_unpack_roundtrip_and_inverse_maps(oracle):
    for W in (16, 32, 64, 128):
        a = np.random.default_rng(W).standard_normal(3 * W * W).astype(np.float32)
        assert np.array_equal(oracle.unpack_weights(oracle.pack_weights(a, 3, W), 3, W), a)
        for idx in (0, 1, W, W + 1, W * W - 1, 5 * W + 3):
            assert oracle.from_packed(oracle.to_packed(idx, W, W), W, W) == idx


def test_packed_transpose_is_transpose_in_packed_layout(oracle):
    for W in (16, 64):
        a = np.random.default_rng(1).standard_normal((W, W)).astype(np.float32)
        pt = oracle.packed_transpose(oracle.pack_weights(a.ravel(), 1, W), W)
        assert np.array_equal(oracle.unpack_weights(pt, 1, W).reshape(W, W), a.T)
        # twice = identity
        assert np.array_equal(oracle.packed_transpose(pt, W), oracle.pack_weights(a.ravel(), 1, W))


def test_pack_and_transpose(oracle):
    W = 32
    raw = np.random.default_rng(2).standard_normal((W, W)).astype(np.float32)  # [out][in]
    p = oracle.pack_and_transpose(raw.ravel(), W)
    assert np.array_equal(oracle.unpack_weights(p, 1, W).reshape(W, W), raw.T)


def test_zero_weights_padding(oracle):
    # include/network/Network.h:171-233 : bias-by-ones keeps rows up to the next multiple of 16
    W, n_mats = 64, 3
    ones = np.ones(n_mats * W * W, np.float32)
    for n_in, n_out, bias, kept_rows in ((3, 5, True, 16), (3, 5, False, 3), (16, 64, True, 64), (33, 1, True, 48), (64, 64, False, 64)):
        z = oracle.unpack_weights(oracle.zero_weights_padding(oracle.pack_weights(ones, n_mats, W), n_mats, W, n_in, n_out, bias), n_mats, W)
        z = z.reshape(n_mats, W, W)
        exp0 = np.zeros((W, W)); exp0[:kept_rows] = 1
        expL = np.zeros((W, W)); expL[:, :n_out] = 1
        assert np.array_equal(z[0], exp0)
        assert np.array_equal(z[1], np.ones((W, W)))
        assert np.array_equal(z[2], expL)
