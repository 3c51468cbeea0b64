"""Pins the oracle's MLP functions: closed forms the reference's tests use, a library routine
(torch linear chain + autograd in fp64), finite differences, and the distance between the
double-precision restatement of test/mlp.h and the restatement of the device rounding points."""
import numpy as np
import pytest
import torch

from oracle_bindings import BF16, FP16

ACTS = ["none", "relu", "sigmoid"]


def torch_act(name):
    return {"none": lambda t: t, "relu": torch.relu, "sigmoid": torch.sigmoid}[name]


def rand_net(W, n_mats, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    lim = scale * np.sqrt(6.0 / (2 * W))
    return rng.uniform(-lim, lim, (n_mats, W, W))


def test_forward_constant_weights_closed_form(oracle):
    # test/doctest_swiftnet.cpp:44-51,79-96: weights 0.01, input 1 on the first n_in columns:
    # hidden = 0.01*n_in, then *W*0.01 per further matrix; padded output columns 0
    W, n_in, n_out, n_mats = 64, 7, 5, 3
    w = np.full((n_mats, W, W), 0.01)
    w[0, n_in:, :] = 0
    w[-1, :, n_out:] = 0
    x = np.zeros((8, W)); x[:, :n_in] = 1.0
    lo = oracle.mlp_forward_f64(W, n_mats, "none", "none", w, x)
    assert np.allclose(lo[1], 0.01 * n_in)
    assert np.allclose(lo[2], 0.01 * n_in * W * 0.01)
    assert np.allclose(lo[3][:, :n_out], 0.01 * n_in * W * 0.01 * W * 0.01)
    assert np.all(lo[3][:, n_out:] == 0)


def test_forward_identity_scaling_closed_form(oracle):
    # benchmarks/benchmark_inference.h:47-48,71: weights 1/W and a constant input reproduce the input
    for W in (16, 32, 64, 128):
        n_mats = 5
        w = np.full((n_mats, W, W), 1.0 / W)
        x = np.full((16, W), 0.37)
        lo = oracle.mlp_forward_f64(W, n_mats, "relu", "none", w, x)
        assert np.allclose(lo, 0.37)
        loT = oracle.mlp_forward_T(BF16, W, n_mats, "relu", "none", oracle.round(w, BF16), oracle.round(x, BF16))
        assert np.allclose(loT, oracle.round(np.float32(0.37), BF16), rtol=2 ** -7)


def test_backward_dw_ones_closed_form(oracle):
    # benchmarks/benchmark_training.h:48-59,90-96: x = dL/dy = sqrt(1/B), w = 1/W, act None => all dW == 1
    W, n_mats, B = 32, 4, 64
    w = np.full((n_mats, W, W), 1.0 / W)
    v = np.sqrt(1.0 / B)
    x = np.full((B, W), v)
    lo = oracle.mlp_forward_f64(W, n_mats, "none", "none", w, x)
    deltas, dW, dX = oracle.mlp_backward_f64(W, n_mats, "none", "none", w, lo, np.full((B, W), v))
    assert np.allclose(lo, v) and np.allclose(deltas, v) and np.allclose(dW, 1.0) and np.allclose(dX, v)


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("out_act", ACTS)
def test_f64_matches_torch_autograd(oracle, act, out_act):
    W, n_mats, M = 16, 3, 24
    w = rand_net(W, n_mats, 3, scale=2.0)
    rng = np.random.default_rng(4)
    x = rng.uniform(-1, 1, (M, W))
    g = rng.standard_normal((M, W))
    lo = oracle.mlp_forward_f64(W, n_mats, act, out_act, w, x)
    deltas, dW, dX = oracle.mlp_backward_f64(W, n_mats, act, out_act, w, lo, g)

    tw = [torch.tensor(w[l], dtype=torch.float64, requires_grad=True) for l in range(n_mats)]
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    h = tx
    pre = []
    for l in range(n_mats):
        z = torch.nn.functional.linear(h, tw[l].T)  # y[n] = sum_k x[k] w[k][n]
        z.retain_grad()
        pre.append(z)
        h = torch_act(out_act if l == n_mats - 1 else act)(z)
        assert np.allclose(h.detach().numpy(), lo[l + 1], atol=1e-12)
    h.backward(torch.tensor(g))
    assert np.allclose(dX, tx.grad.numpy(), atol=1e-12)
    for l in range(n_mats):
        assert np.allclose(deltas[l], pre[l].grad.numpy(), atol=1e-12)
        # dW layout is [n=out][k=in]
        assert np.allclose(dW[l], tw[l].grad.numpy().T, atol=1e-11)


def test_f64_backward_finite_differences(oracle):
    W, n_mats, M = 16, 2, 8
    w = rand_net(W, n_mats, 5, scale=2.0)
    rng = np.random.default_rng(6)
    x = rng.uniform(-1, 1, (M, W))
    g = rng.standard_normal((M, W))

    def loss(wv, xv):
        return float((oracle.mlp_forward_f64(W, n_mats, "sigmoid", "none", wv, xv)[-1] * g).sum())

    lo = oracle.mlp_forward_f64(W, n_mats, "sigmoid", "none", w, x)
    _, dW, dX = oracle.mlp_backward_f64(W, n_mats, "sigmoid", "none", w, lo, g)
    eps = 1e-6
    for (l, k, n) in ((0, 3, 5), (1, 0, 15), (1, 7, 7)):
        wp, wm = w.copy(), w.copy()
        wp[l, k, n] += eps
        wm[l, k, n] -= eps
        fd = (loss(wp, x) - loss(wm, x)) / (2 * eps)
        assert abs(fd - dW[l, n, k]) < 1e-6 * max(1, abs(fd))
    xp, xm = x.copy(), x.copy()
    xp[2, 4] += eps
    xm[2, 4] -= eps
    assert abs((loss(w, xp) - loss(w, xm)) / (2 * eps) - dX[2, 4]) < 1e-6


@pytest.mark.parametrize("dtype,tol", [(BF16, 1e-2), (FP16, 2e-3)])
@pytest.mark.parametrize("act,out_act", [("relu", "none"), ("none", "none"), ("sigmoid", "sigmoid"), ("relu", "relu")])
def test_T_restatement_close_to_f64(oracle, dtype, tol, act, out_act):
    """The rounding-point restatement (kernel_esimd.h) stays within the reference's own 1e-2
    max-norm tolerance (result_check.h:83-102) of the double oracle (mlp.h)."""
    W, n_mats, M = 64, 5, 256
    rng = np.random.default_rng(7)
    w = oracle.round(rand_net(W, n_mats, 8), dtype)
    x = oracle.round(rng.uniform(-1, 1, (M, W)), dtype)
    # fp16 gradients carry the reference's loss scale of 128 (dpcpp_bindings/tiny_dpcpp_nn/modules.py:158-161),
    # which keeps the deltas out of the fp16 denormal range
    g = oracle.round(rng.uniform(-1, 1, (M, W)) / M * (128.0 if dtype == FP16 else 1.0), dtype)
    lo = oracle.mlp_forward_f64(W, n_mats, act, out_act, w, x)
    loT = oracle.mlp_forward_T(dtype, W, n_mats, act, out_act, w, x)

    def rel(a, b):
        return np.abs(a - b).max() / max(np.abs(a).max(), np.abs(b).max(), 1e-30)

    for l in range(n_mats + 1):
        assert rel(loT[l], lo[l]) < tol
    deltas, dW, dX = oracle.mlp_backward_f64(W, n_mats, act, out_act, w, lo, g)
    # as in test/doctest_swiftnet.cpp:176,192 the backward is fed the reference forward activations, so
    # that ReLU masks of near-zero activations do not differ between the two
    ib, dWT, dXT = oracle.mlp_backward_T(dtype, W, n_mats, act, out_act, w, oracle.round(lo, dtype), g)
    for l in range(n_mats):
        assert rel(ib[l], deltas[l]) < 2 * tol
        assert rel(dWT[l], dW[l]) < 2 * tol
    assert rel(dXT, dX) < 2 * tol


def test_T_restatement_exact_when_nothing_rounds(oracle):
    """Small-integer weights and inputs: every product and sum is exactly representable in bf16, so
    the rounding-point restatement must equal the double oracle bit for bit."""
    W, n_mats, M = 16, 2, 8
    rng = np.random.default_rng(9)
    w = rng.integers(-1, 2, (n_mats, W, W)).astype(np.float64) * 0.5
    x = rng.integers(-2, 3, (M, W)).astype(np.float64)
    g = rng.integers(-2, 3, (M, W)).astype(np.float64)
    lo = oracle.mlp_forward_f64(W, n_mats, "relu", "none", w, x)
    assert np.abs(lo).max() < 128  # 8 significant bits are enough for multiples of 0.25 below 64; check below
    loT = oracle.mlp_forward_T(BF16, W, n_mats, "relu", "none", w, x)
    exact = oracle.round(lo, BF16) == lo.astype(np.float32)
    assert np.array_equal(loT[exact], lo.astype(np.float32)[exact])
    assert exact.mean() > 0.9
    # fp16 has 11 significant bits: everything here is exact
    loH = oracle.mlp_forward_T(FP16, W, n_mats, "relu", "none", w, x)
    assert np.array_equal(loH, lo.astype(np.float32))
    deltas, dW, dX = oracle.mlp_backward_f64(W, n_mats, "relu", "none", w, lo, g)
    ib, dWH, dXH = oracle.mlp_backward_T(FP16, W, n_mats, "relu", "none", w, loH, g)
    assert np.array_equal(ib, deltas.astype(np.float32))
    assert np.array_equal(dXH, dX.astype(np.float32))
    assert np.array_equal(dWH, oracle.round(dW, FP16))


def test_rounding_helpers(oracle):
    v = np.array([1.0, 1.00390625, 1.005859375, 3.14159265, -2.7182818, 1e-40, 65504.0, 65520.0, 6e-8, 5.9604645e-08, 0.0], np.float32)
    tb = torch.tensor(v).to(torch.bfloat16).to(torch.float32).numpy()
    th = torch.tensor(v).to(torch.float16).to(torch.float32).numpy()
    assert np.array_equal(oracle.round(v, BF16), tb)
    assert np.array_equal(oracle.round(v, FP16), th)
    r = np.random.default_rng(0).standard_normal(100000).astype(np.float32) * np.float32(10.0) ** np.random.default_rng(1).integers(-9, 5, 100000)
    assert np.array_equal(oracle.round(r, BF16), torch.tensor(r).to(torch.bfloat16).to(torch.float32).numpy())
    assert np.array_equal(oracle.round(r, FP16), torch.tensor(r).to(torch.float16).to(torch.float32).numpy())
