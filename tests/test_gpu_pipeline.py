"""BASELINE configs 4 and 5 end to end through the C ABI: hash-grid encoding feeding the fused MLP.

Config 5 (3-D grid -> width-64 MLP with 3 hidden layers, 16 outputs, inference): the GPU chain tnn_grid_forward (fp16 table,
fp16 output padded to the network width) -> tnn_mlp_inference against the oracle's chain on the same seeded inputs.
Config 4 (2-D grid -> width-64 MLP with 2 hidden layers, 3 outputs, full training step with backward into the table): encoding,
fused training step (forward, L2 loss, backward, weight gradients, dL/d(encoding)), scatter into the gradient table, Adam on both
parameter sets, against the same steps done by the oracle.

Tolerances (tests/tolerances.py): fp16 5e-3 relative with an absolute floor scaled to the quantity's size; "propagated" where a
value went through several rounded layers; gradient-table entries are sums of fp32 atomics in arbitrary order.
"""
import ctypes

import numpy as np
import pytest
import torch

from gpu_harness import ptr
from tiny_dpcpp_nn import _lib
from tolerances import FP16, FP32, assert_close, assert_propagated, max_norm_rel

pytestmark = pytest.mark.gpu

CFG4 = dict(n_dims=2, n_levels=16, n_features_per_level=2, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.5)
CFG5 = dict(n_dims=3, n_levels=16, n_features_per_level=2, log2_hashmap_size=22, base_resolution=16, per_level_scale=1.447)
W = 64


def xavier(rng, n_mats, n_in, n_out):
    """Unpacked [in][out] matrices, Xavier-uniform, rows / columns that only see padding zeroed (what
    Network::ZeroWeightsPadding leaves, include/network/Network.h:171-233 of the reference)."""
    lim = np.sqrt(6.0 / (2 * W))
    w = rng.uniform(-lim, lim, (n_mats, W, W)).astype(np.float32)
    w[0, n_in:, :] = 0
    w[-1, :, n_out:] = 0
    return w


@pytest.mark.parametrize("M", [1 << 14, 1 << 21])
def test_config_5_encoding_plus_mlp_inference(tnn, oracle, M):
    """At 2^14 points every output is compared; at the full 2^21 the oracle chain runs on a seeded sample of 2^14 rows and the
    padded output columns (zero weights) are checked on every row."""
    n_hidden, n_out = 3, 16
    n_mats = n_hidden + 1
    rng = np.random.default_rng(55)
    gd = tnn.grid_desc(CFG5, FP16)
    n = tnn.grid_n_params(gd)
    gen = torch.Generator(device=tnn.dev).manual_seed(55)
    # the table of the config is U(+-1e-4); a wider one is used here so that the network sees inputs of ordinary size
    table = (torch.rand(n, device=tnn.dev, generator=gen) * 2 - 1).to(torch.float16)
    x = torch.rand((M, 3), device=tnn.dev, generator=gen)
    w = oracle.round(xavier(rng, n_mats, 32, n_out), FP16)
    desc = tnn.mlp_desc(FP16, W, n_hidden, "relu", "none")
    _, pf, _ = tnn.prepare(desc, w)

    enc = tnn.grid_forward(gd, x, table, W, FP16)
    y = tnn.inference(desc, pf, enc)
    assert y.shape == (M, W)
    assert bool((y[:, n_out:] == 0).all())
    assert bool((enc[:, 32:] == 0).all())

    sel = np.arange(M) if M <= (1 << 14) else np.sort(rng.choice(M, 1 << 14, replace=False))
    xs = x.cpu().numpy()[sel]
    enc_ref = oracle.round(oracle.grid_forward(CFG5, table.float().cpu().numpy(), xs, W), FP16)
    assert_close(enc.float().cpu().numpy()[sel], enc_ref, FP16, "encoding")
    y_ref = oracle.mlp_forward_T(FP16, W, n_mats, "relu", "none", w, enc_ref, store_interm=False)
    assert_propagated(y.float().cpu().numpy()[sel], y_ref, FP16, "network output")


@pytest.mark.parametrize("M", [1 << 13, 1 << 18])
def test_config_4_training_step_with_table_gradients(tnn, oracle, M):
    """One full optimisation step of config 4. The loss of the config is the mean over the 3 real outputs; the fused step
    averages over the padded width, so the loss scale carries the factor W / 3 (targets and outputs of the padded columns are
    both zero and add nothing)."""
    n_hidden, n_out = 2, 3
    n_mats = n_hidden + 1
    rng = np.random.default_rng(44)
    gd = tnn.grid_desc(CFG4, FP16)
    n_table = tnn.grid_n_params(gd)
    gen = torch.Generator(device=tnn.dev).manual_seed(44)
    table_master = torch.rand(n_table, device=tnn.dev, generator=gen) * 2 - 1
    table = table_master.to(torch.float16)
    x = torch.rand((M, 2), device=tnn.dev, generator=gen)
    targets = torch.zeros((M, W), device=tnn.dev)
    targets[:, :n_out] = torch.rand((M, n_out), device=tnn.dev, generator=gen)
    w = oracle.round(xavier(rng, n_mats, 32, n_out), FP16)
    desc = tnn.mlp_desc(FP16, W, n_hidden, "relu", "none")
    # 128 at 2^13 rows, growing with the batch: dL/dy = loss_scale * 2 (y - t) / (M W) then keeps its size, clear of fp16's
    # denormal range (at 2^18 rows a scale of 128 leaves most of dL/d(encoding) within a few denormal steps of zero)
    loss_scale = 128.0 * W / n_out * (M / 8192)

    # ---- GPU: encode, fused step (with dL/d(encoding)), scatter, Adam on both parameter sets
    master = tnn.pack(FP32, W, n_mats, torch.from_numpy(w.reshape(-1)).to(tnn.dev))
    pf, pb = tnn.prepare_packed(desc, master, src_is_fp32=True)
    enc = tnn.grid_forward(gd, x, table, W, FP16)
    y, loss, dW, dEnc = tnn.train_step_l2(desc, pf, pb, enc, targets, loss_scale, want_y=True, want_dx=True, dw_fp32=True)
    grad_table = tnn.grid_backward(gd, x, dEnc, FP16)
    table_before, master_before = table_master.clone(), master.clone()
    m_w, v_w = torch.zeros_like(master), torch.zeros_like(master)
    hyper = (1e-3, 0.9, 0.99, 1e-15)
    _lib.check(tnn.lib.tnn_mlp_adam_update(ctypes.byref(desc), ptr(master), ptr(m_w), ptr(v_w), ptr(dW), 1.0 / loss_scale, 1, *hyper,
                                           None, ptr(pf), ptr(pb), tnn.stream()))
    m_t, v_t = torch.zeros_like(table_master), torch.zeros_like(table_master)
    tnn.adam_step(table_master, m_t, v_t, grad_table, FP32, 1.0 / loss_scale, 1, *hyper, table, FP16)

    # ---- oracle: the same steps
    xs = x.cpu().numpy()
    enc_ref = oracle.round(oracle.grid_forward(CFG4, table_before.to(torch.float16).float().cpu().numpy(), xs, W), FP16)
    assert_close(enc.float().cpu().numpy(), enc_ref, FP16, "encoding")
    interm = oracle.mlp_forward_T(FP16, W, n_mats, "relu", "none", w, enc_ref)
    assert_propagated(y.float().cpu().numpy(), interm[-1], FP16, "network output")
    values, grads = oracle.l2_loss(FP16, interm[-1], targets.cpu().numpy(), loss_scale)
    assert abs(float(loss.item()) - float(values.sum())) <= 1e-3 * float(values.sum())
    _, dW_ref, dEnc_ref = oracle.mlp_backward_T(FP16, W, n_mats, "relu", "none", w, interm, grads, round_dw=False)
    assert_propagated(dW.cpu().numpy(), dW_ref, FP16, "dW", scale=float(np.abs(dW_ref).max()))
    dEnc_h = dEnc.float().cpu().numpy()
    # 16.7 million values behind two ReLU layers: where the GPU's and the oracle's fp32 sums round a pre-activation to
    # different sides of zero the mask flips and the element moves by a whole term, not by a rounding step. The bar of the
    # other propagated quantities (0.2 % outside), with ten elements in a million allowed beyond four times the bar
    # instead of none, and the error of the whole matrix in the Frobenius norm in place of the max norm (which a single
    # flipped element decides).
    top = float(np.abs(dEnc_ref).max())
    diff, bar = np.abs(dEnc_h - dEnc_ref), 5e-4 * top + 5e-3 * np.abs(dEnc_ref)
    outside, far = float((diff > bar).mean()), float((diff > 4 * bar).mean())
    assert outside <= 2e-3 and far <= 1e-5, (outside, far)
    assert np.linalg.norm((dEnc_h - dEnc_ref).ravel()) <= 5e-3 * np.linalg.norm(dEnc_ref.ravel())
    # the scatter is checked on the GPU's own dL/d(encoding), so that only this step is compared
    gt_ref = oracle.grid_backward(CFG4, xs, dEnc_h, n_table)
    gt = grad_table.cpu().numpy()
    assert np.abs(gt - gt_ref).max() <= 1e-5 * np.abs(gt_ref).max() + 1e-6
    assert max_norm_rel(gt, gt_ref) <= 1e-5
    # Adam on both parameter sets, from the GPU's own gradients (step 1, zero moments)
    g_t = gt / loss_scale
    p_ref, _, _ = oracle.adam_step(table_before.cpu().numpy(), np.zeros(n_table, np.float32), np.zeros(n_table, np.float32), g_t, 1, *hyper)
    assert np.allclose(table_master.cpu().numpy(), p_ref, rtol=1e-6, atol=1e-7)
    assert np.array_equal(table.float().cpu().numpy(), oracle.round(table_master.cpu().numpy(), FP16))
    dW_h = dW.cpu().numpy()
    dW_packed = np.stack([oracle.pack_and_transpose(dW_h[l], W) for l in range(n_mats)]).reshape(-1) / loss_scale
    n_w = n_mats * W * W
    pw_ref, _, _ = oracle.adam_step(master_before.cpu().numpy(), np.zeros(n_w, np.float32), np.zeros(n_w, np.float32), dW_packed, 1, *hyper)
    assert np.allclose(master.cpu().numpy(), pw_ref, rtol=1e-6, atol=1e-7)
    # weights that only see padding had zero gradients and stayed zero
    unp = oracle.unpack_weights(master.cpu().numpy(), n_mats, W).reshape(n_mats, W, W)
    assert np.all(unp[0, 32:, :] == 0) and np.all(unp[-1, :, n_out:] == 0)
