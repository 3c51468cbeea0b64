"""tnn_grid_mlp_train_step_l2_adam: hash-grid encoding, network forward, L2 loss, backward pass, Adam on the network and the
scatter into the table's gradient, with the encoding evaluated inside the training kernel.

Bar: the three-call chain tnn_grid_forward (output in the network's type, padded to its width) -> tnn_mlp_train_step_l2_adam
(with dL/dx) -> tnn_grid_backward, whose kernels are checked against the oracle elsewhere. The fused kernel blends, rounds,
multiplies and reduces in the same order: network output, loss, Adam state and the re-staged weights must be equal bit for
bit. The table's gradient is a sum of fp32 atomics in no defined order: |a - b| <= 1e-5 x the largest entry, the bar of
tnn_grid_backward against the oracle. One case checks the gradient against the oracle's scatter of the chain's dL/d(encoding)
directly.
"""
import ctypes

import numpy as np
import pytest
import torch

from gpu_harness import BF16, FP16, FP32, ptr
from tiny_dpcpp_nn import _lib

pytestmark = pytest.mark.gpu
HYPER = (1e-2, 0.9, 0.99, 1e-8)


def setup(tnn, cfg, table_dtype, dtype, n_hidden, M, seed, n_out=3, out_act="none"):
    W = 64
    rng = np.random.default_rng(seed)
    gd = tnn.grid_desc(cfg, table_dtype)
    n = tnn.grid_n_params(gd)
    gen = torch.Generator(device=tnn.dev).manual_seed(seed)
    table = (torch.rand(n, device=tnn.dev, generator=gen) * 2 - 1).to(torch.float16 if table_dtype == FP16 else torch.float32)
    x = torch.rand((M, cfg["n_dims"]), device=tnn.dev, generator=gen)
    targets = torch.zeros((M, W), device=tnn.dev)
    targets[:, :n_out] = torch.rand((M, n_out), device=tnn.dev, generator=gen)
    n_feat = cfg["n_levels"] * cfg["n_features_per_level"]
    lim = np.sqrt(6.0 / (2 * W))
    w = rng.uniform(-lim, lim, (n_hidden + 1, W, W)).astype(np.float32)
    w[0, n_feat:, :] = 0
    w[-1, :, n_out:] = 0
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", out_act)
    master = tnn.pack(FP32, W, n_hidden + 1, torch.from_numpy(w.reshape(-1)).to(tnn.dev))
    return dict(gd=gd, n=n, table=table, x=x, targets=targets, desc=desc, master=master, W=W, M=M, dtype=dtype)


def state(tnn, c):
    master = c["master"].clone()
    pf, pb = tnn.prepare_packed(c["desc"], master, src_is_fp32=True)
    return dict(master=master, pf=pf, pb=pb, m=torch.zeros_like(master), v=torch.zeros_like(master),
                loss=torch.full((1,), float("nan"), device=tnn.dev),
                y=torch.full((c["M"], c["W"]), float("nan"), dtype=torch.bfloat16 if c["dtype"] == BF16 else torch.float16, device=tnn.dev))


def chain_step(tnn, c, st, step, loss_scale, grad, overwrite, ordered):
    L, M, W = tnn.lib, c["M"], c["W"]
    md, g = ctypes.byref(c["desc"]), c["gd"]
    order = tnn.grid_order(g, c["x"]) if ordered else None
    enc = tnn.grid_forward_ordered(g, order, c["table"], W, M, c["dtype"]) if ordered else tnn.grid_forward(g, c["x"], c["table"], W, c["dtype"])
    d_enc = torch.empty_like(enc)
    ws_bytes = L.tnn_mlp_train_step_workspace_bytes(md, M)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=tnn.dev)
    _lib.check(L.tnn_mlp_train_step_l2_adam(md, ptr(st["pf"]), ptr(st["pb"]), ptr(enc), ptr(c["targets"]), loss_scale, ptr(st["y"]), ptr(st["loss"]),
                                            ptr(st["master"]), ptr(st["m"]), ptr(st["v"]), step, *HYPER, None, ptr(d_enc), M, ptr(ws), ws_bytes, None,
                                            tnn.stream()))
    if ordered:
        tnn.grid_backward_ordered(g, order, d_enc, c["dtype"], grad_t=grad, overwrite=overwrite)
    else:
        tnn.grid_backward(g, c["x"], d_enc, c["dtype"], grad_t=grad, overwrite=overwrite)
    return d_enc


def fused_step(tnn, c, st, step, loss_scale, grad, overwrite, ordered):
    L, M = tnn.lib, c["M"]
    md, g = ctypes.byref(c["desc"]), ctypes.byref(c["gd"])
    assert L.tnn_grid_mlp_train_supported(g, md) == _lib.TNN_OK
    order = tnn.grid_order(c["gd"], c["x"]) if ordered else None
    ws_bytes = L.tnn_grid_mlp_train_step_workspace_bytes(g, md, M)
    assert ws_bytes > 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=tnn.dev)
    _lib.check(L.tnn_grid_mlp_train_step_l2_adam(g, md, None if ordered else ptr(c["x"]), ptr(order) if ordered else None, ptr(c["table"]),
                                                 ptr(st["pf"]), ptr(st["pb"]), ptr(c["targets"]), loss_scale, ptr(st["y"]), ptr(st["loss"]),
                                                 ptr(st["master"]), ptr(st["m"]), ptr(st["v"]), step, *HYPER, None, ptr(grad), int(overwrite), M,
                                                 ptr(ws), ws_bytes, tnn.stream()))


def bits(t):
    return t.contiguous().view(torch.uint8)


def same_state(a, b, ordered, what):
    """Caller's order: everything bit for bit. Cell order: the fused kernel's tiles hold other rows than the chain's, so the
    fp32 sums over the batch (weight gradients, loss) are taken in another order: per-row results stay bit-equal, the sums
    and what Adam makes of them agree to fp32 rounding, the re-staged weights to an ulp of the network's type."""
    assert torch.equal(bits(a["y"]), bits(b["y"])), f"y differs, {what}"
    if not ordered:
        for k in ("loss", "master", "m", "v", "pf", "pb"):
            assert torch.equal(bits(a[k]), bits(b[k])), f"{k} differs, {what}"
        return
    assert abs(float(a["loss"]) - float(b["loss"])) <= 1e-5 * abs(float(a["loss"])), what
    for k, rtol, atol in (("m", 1e-3, 1e-7), ("v", 1e-3, 1e-12), ("master", 1e-5, 2e-6)):
        assert torch.allclose(a[k], b[k], rtol=rtol, atol=atol), f"{k}, {what}: {float((a[k] - b[k]).abs().max())}"
    for k in ("pf", "pb"):
        assert torch.allclose(a[k].float(), b[k].float(), rtol=2 ** -7, atol=1e-5), f"{k}, {what}"
        assert float((bits(a[k]) != bits(b[k])).float().mean()) < 0.01, f"{k}, {what}: too many weights rounded the other way"


CASES = [
    # dims, levels, log2_hashmap, base, scale, table, net type, hidden, M, out_act
    (2, 16, 15, 16, 1.5, FP16, FP16, 2, 8192, "none"),    # BASELINE config 4's shape, small table
    (2, 16, 15, 16, 1.5, FP16, FP16, 2, 4104, "none"),    # ragged last tile, fewer tiles than waves in the last round
    (3, 16, 15, 16, 1.447, FP16, FP16, 3, 2048 * 9, "none"),  # config 5's shape, several rounds per wave
    (3, 12, 14, 8, 1.6, FP32, BF16, 4, 3000 * 8, "relu"),  # fp32 table, bf16 network, deepest supported, 24 of 32 pieces real
    (2, 5, 12, 16, 2.0, FP32, BF16, 1, 8, "sigmoid"),     # one tile of 8 rows, a piece that is half real
    (2, 32, 10, 4, 1.2, FP16, FP16, 2, 4096, "none"),     # 32 levels: every column of the width-64 input is an encoded feature
    (3, 27, 11, 4, 1.25, FP32, BF16, 3, 2056, "none"),    # more than 22 levels, last piece not full
]


@pytest.mark.parametrize("ordered", [False, True])
@pytest.mark.parametrize("case", CASES)
def test_fused_step_equals_the_three_calls(tnn, case, ordered):
    D, L_, log2, base, scale, tdt, dt, n_hidden, M, out_act = case
    cfg = dict(n_dims=D, n_levels=L_, n_features_per_level=2, log2_hashmap_size=log2, base_resolution=base, per_level_scale=scale)
    c = setup(tnn, cfg, tdt, dt, n_hidden, M, seed=M + D, out_act=out_act)
    a, b = state(tnn, c), state(tnn, c)
    ga = torch.full((c["n"],), 0.5, device=tnn.dev)
    gb = ga.clone()
    loss_scale = 128.0
    for step in (1, 2, 3):  # the first overwrites the table's gradient, the others accumulate
        chain_step(tnn, c, a, step, loss_scale, ga, step == 1, ordered)
        fused_step(tnn, c, b, step, loss_scale, gb, step == 1, ordered)
        tnn.sync()
        same_state(a, b, ordered, f"step {step}")
        assert bool(torch.isfinite(b["loss"]).all()) and float(b["loss"]) > 0
        ref = ga.cpu().numpy()
        assert np.abs(gb.cpu().numpy() - ref).max() <= 1e-5 * max(1.0, np.abs(ref).max()), f"table gradient at step {step}"
    assert float(ga.abs().max()) > 0


def test_table_gradient_against_the_oracle(tnn, oracle):
    cfg = dict(n_dims=2, n_levels=16, n_features_per_level=2, log2_hashmap_size=15, base_resolution=16, per_level_scale=1.5)
    c = setup(tnn, cfg, FP16, FP16, 2, 8192, seed=5)
    a, b = state(tnn, c), state(tnn, c)
    ga, gb = torch.zeros(c["n"], device=tnn.dev), torch.zeros(c["n"], device=tnn.dev)
    d_enc = chain_step(tnn, c, a, 1, 64.0, ga, True, False)
    fused_step(tnn, c, b, 1, 64.0, gb, True, True)
    tnn.sync()
    ref = oracle.grid_backward(cfg, c["x"].cpu().numpy(), d_enc.float().cpu().numpy(), c["n"])
    assert np.abs(gb.cpu().numpy() - ref).max() <= 1e-5 * max(1.0, np.abs(ref).max())


def test_config_4_full_size(tnn):
    """BASELINE config 4 at its batch size (2^18 points, 2^19-entry levels): fused against the three calls."""
    cfg = dict(n_dims=2, n_levels=16, n_features_per_level=2, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.5)
    c = setup(tnn, cfg, FP16, FP16, 2, 1 << 18, seed=11)
    a, b = state(tnn, c), state(tnn, c)
    ga, gb = torch.zeros(c["n"], device=tnn.dev), torch.zeros(c["n"], device=tnn.dev)
    loss_scale = 128.0 * 64 / 3 * 32
    chain_step(tnn, c, a, 1, loss_scale, ga, True, True)
    fused_step(tnn, c, b, 1, loss_scale, gb, True, True)
    tnn.sync()
    same_state(a, b, True, "config 4")
    ref = ga.cpu().numpy()
    assert np.abs(gb.cpu().numpy() - ref).max() <= 1e-5 * max(1.0, np.abs(ref).max())


def test_rejects_what_it_cannot_run(tnn):
    L = tnn.lib
    g2 = tnn.grid_desc(dict(n_dims=2, n_levels=8, n_features_per_level=2, log2_hashmap_size=12, base_resolution=16, per_level_scale=1.5), FP16)
    g4 = tnn.grid_desc(dict(n_dims=2, n_levels=8, n_features_per_level=4, log2_hashmap_size=12, base_resolution=16, per_level_scale=1.5), FP16)
    ok = tnn.mlp_desc(FP16, 64, 2, "relu", "none")
    for gd, md in ((g4, ok), (g2, tnn.mlp_desc(FP16, 32, 2, "relu", "none")), (g2, tnn.mlp_desc(FP16, 64, 2, "sigmoid", "none")),
                   (g2, tnn.mlp_desc(FP16, 64, 5, "relu", "none"))):
        assert L.tnn_grid_mlp_train_supported(ctypes.byref(gd), ctypes.byref(md)) == _lib.TNN_ERR_UNSUPPORTED
        assert L.tnn_grid_mlp_train_step_workspace_bytes(ctypes.byref(gd), ctypes.byref(md), 1024) == 0
    # too many levels for the network's width
    g40 = tnn.grid_desc(dict(n_dims=2, n_levels=40, n_features_per_level=2, log2_hashmap_size=10, base_resolution=4, per_level_scale=1.1), FP16)
    assert L.tnn_grid_mlp_train_supported(ctypes.byref(g40), ctypes.byref(ok)) < 0
    z = torch.zeros(64, device=tnn.dev)
    rc = L.tnn_grid_mlp_train_step_l2_adam(ctypes.byref(g2), ctypes.byref(ok), ptr(z), None, ptr(z), ptr(z), ptr(z), ptr(z), 1.0, None, None, ptr(z),
                                           ptr(z), ptr(z), 1, *HYPER, None, ptr(z), 1, 12, None, 0, None)
    assert rc == _lib.TNN_ERR_INVALID_ARGUMENT  # batch not a multiple of 8
    rc = L.tnn_grid_mlp_train_step_l2_adam(ctypes.byref(g2), ctypes.byref(ok), ptr(z), None, ptr(z), ptr(z), ptr(z), ptr(z), 1.0, None, None, ptr(z),
                                           ptr(z), ptr(z), 1, *HYPER, None, ptr(z), 1, 16, None, 0, None)
    assert rc == _lib.TNN_ERR_WORKSPACE
