"""tnn_grid_mlp_inference: the grid encoding feeding the fused MLP inside one kernel.

Two bars. (1) Bit-equality with the two-call chain tnn_grid_forward (output in the network's type, padded to its width) ->
tnn_mlp_inference, whose kernels are themselves checked against the oracle elsewhere: the fused kernel blends, rounds and
multiplies in the same order, so nothing may differ. (2) The oracle's chain directly, on seeded inputs, to the tolerances of
the network's type (tests/tolerances.py), so the check does not rest on the other GPU kernels alone.
"""
import ctypes

import numpy as np
import pytest
import torch

from gpu_harness import BF16, FP16, FP32, ptr
from tiny_dpcpp_nn import _lib
from tolerances import assert_close, assert_propagated

pytestmark = pytest.mark.gpu


def weights(rng, n_mats, W, n_in, n_out):
    lim = np.sqrt(6.0 / (2 * W))
    w = rng.uniform(-lim, lim, (n_mats, W, W)).astype(np.float32)
    w[0, n_in:, :] = 0
    w[-1, :, n_out:] = 0
    return w


def chain_and_fused(tnn, cfg, table_dtype, dtype, W, n_hidden, act, out_act, M, seed, w=None):
    rng = np.random.default_rng(seed)
    gd = tnn.grid_desc(cfg, table_dtype)
    n = tnn.grid_n_params(gd)
    gen = torch.Generator(device=tnn.dev).manual_seed(seed)
    table = (torch.rand(n, device=tnn.dev, generator=gen) * 2 - 1).to(torch.float16 if table_dtype == FP16 else torch.float32)
    x = torch.rand((M, cfg["n_dims"]), device=tnn.dev, generator=gen)
    n_feat = cfg["n_levels"] * cfg["n_features_per_level"]
    if w is None:
        w = weights(rng, n_hidden + 1, W, n_feat, W)
    desc = tnn.mlp_desc(dtype, W, n_hidden, act, out_act)
    _, pf, _ = tnn.prepare(desc, w)
    enc = tnn.grid_forward(gd, x, table, W, dtype)
    y_chain = tnn.inference(desc, pf, enc)
    y_fused = tnn.grid_mlp_inference(gd, desc, x, table, pf)
    # the same kernel over the points in cell order writes the same rows
    y_ordered = tnn.grid_mlp_inference_ordered(gd, desc, tnn.grid_order(gd, x), table, pf, M)
    tnn.sync()
    assert same_bits(y_ordered, y_fused), "cell order changed the fused kernel's result"
    return dict(gd=gd, table=table, x=x, w=w, desc=desc, enc=enc, y_chain=y_chain, y_fused=y_fused)


def same_bits(a, b):
    return bool((a.view(torch.int16) == b.view(torch.int16)).all())


CASES = [
    # dims, levels, F, log2_hashmap, base, scale, table, net type, W, hidden, act, out_act, M
    (3, 16, 2, 15, 16, 1.447, FP16, FP16, 64, 3, "relu", "none", 8192),       # BASELINE config 5's shape, small table
    (2, 16, 2, 15, 16, 1.5, FP16, FP16, 64, 2, "relu", "none", 4104),         # config 4's shape; ragged last tile
    (3, 8, 4, 14, 8, 2.0, FP32, BF16, 32, 2, "relu", "sigmoid", 2048),        # fp32 table, bf16 network, full width
    (2, 12, 1, 12, 4, 1.6, FP32, FP16, 16, 1, "sigmoid", "none", 1032),       # 8 levels per piece, 12 of 16 columns real
    (3, 5, 8, 13, 8, 1.9, FP16, BF16, 64, 4, "none", "relu", 2056),           # one level per piece, 40 of 64 columns real
    (2, 3, 2, 10, 16, 2.0, FP16, FP16, 16, 2, "relu", "none", 8),             # a piece that is half real, a single tile of 8 rows
    (3, 16, 2, 16, 16, 1.447, FP16, FP16, 128, 3, "relu", "none", 1024),      # width 128 (4 matrices fit LDS)
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"d{c[0]}_l{c[1]}_f{c[2]}_w{c[8]}_M{c[12]}")
def test_fused_equals_two_calls_bitwise_and_oracle(tnn, oracle, case):
    D, L, F, log2, base, scale, tdt, dt, W, n_hidden, act, out_act, M = case
    cfg = dict(n_dims=D, n_levels=L, n_features_per_level=F, log2_hashmap_size=log2, base_resolution=base, per_level_scale=scale)
    r = chain_and_fused(tnn, cfg, tdt, dt, W, n_hidden, act, out_act, M, seed=1000 + M)
    assert not bool(torch.isnan(r["y_fused"].float()).any())
    assert same_bits(r["y_fused"], r["y_chain"])
    # the oracle's chain on the same inputs
    w_r = oracle.round(r["w"], dt)
    enc_ref = oracle.round(oracle.grid_forward(cfg, r["table"].float().cpu().numpy(), r["x"].cpu().numpy(), W), dt)
    assert_close(r["enc"].float().cpu().numpy(), enc_ref, dt, "encoding")
    y_ref = oracle.mlp_forward_T(dt, W, n_hidden + 1, act, out_act, w_r, enc_ref, store_interm=False)
    assert_propagated(r["y_fused"].float().cpu().numpy(), y_ref, dt, "network output")


@pytest.mark.parametrize("interp, hash_type, grid_type", [("Smoothstep", "Prime", "Hash"), ("Nearest", "ReversedPrime", "Hash"),
                                                          ("Linear", "CoherentPrime", "Dense"), ("Linear", "CoherentPrime", "Tiled")])
def test_fused_other_grid_variants(tnn, interp, hash_type, grid_type):
    cfg = dict(n_dims=3, n_levels=8, n_features_per_level=2, log2_hashmap_size=12, base_resolution=4, per_level_scale=1.5,
               interpolation=interp, hash=hash_type, grid_type=grid_type)
    r = chain_and_fused(tnn, cfg, FP16, FP16, 32, 2, "relu", "none", 4096, seed=7)
    assert same_bits(r["y_fused"], r["y_chain"])


def test_fused_config_5_full_size(tnn):
    """2^21 points, 2^22-entry hash levels (162 MiB table): bit-equality with the chain on every row."""
    cfg = dict(n_dims=3, n_levels=16, n_features_per_level=2, log2_hashmap_size=22, base_resolution=16, per_level_scale=1.447)
    rng = np.random.default_rng(5)
    w = weights(rng, 4, 64, 32, 16)
    r = chain_and_fused(tnn, cfg, FP16, FP16, 64, 3, "relu", "none", 1 << 21, seed=5, w=w)
    assert same_bits(r["y_fused"], r["y_chain"])
    assert bool((r["y_fused"][:, 16:] == 0).all())


def test_fused_rejects_what_it_cannot_run(tnn):
    cfg = dict(n_dims=3, n_levels=16, n_features_per_level=2, log2_hashmap_size=12, base_resolution=4, per_level_scale=1.5)
    gd = tnn.grid_desc(cfg, FP16)
    table = torch.zeros(tnn.grid_n_params(gd), dtype=torch.float16, device=tnn.dev)
    x = torch.zeros((64, 3), device=tnn.dev)

    def call(desc, M=64):
        nbytes = tnn.lib.tnn_mlp_prepared_bytes(ctypes.byref(desc))
        pf = torch.zeros(nbytes // 2, dtype=torch.float16, device=tnn.dev)
        y = torch.zeros((64, desc.width), dtype=torch.float16, device=tnn.dev)
        return tnn.lib.tnn_grid_mlp_inference(ctypes.byref(gd), ctypes.byref(desc), ptr(x), ptr(table), ptr(pf), ptr(y), M, tnn.stream())

    # 32 encoded features do not fit a width-16 network (include/encodings/grid.h:665-677)
    assert call(tnn.mlp_desc(FP16, 16, 2, "relu", "none")) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert b"Dimension mismatch" in tnn.lib.tnn_last_error()
    # width 128 with 9 matrices: 288 KiB of weights, more than LDS holds
    assert call(tnn.mlp_desc(FP16, 128, 8, "relu", "none")) == _lib.TNN_ERR_UNSUPPORTED
    # batch not a multiple of 8 (include/network/SwiftNetMLP.h:293-300)
    assert call(tnn.mlp_desc(FP16, 64, 2, "relu", "none"), M=60) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert call(tnn.mlp_desc(FP16, 64, 2, "relu", "none")) == _lib.TNN_OK
    tnn.sync()
