"""L2 loss closed form and Adam against torch.optim.Adam (the optimizer the reference's loops use)."""
import numpy as np
import torch

from oracle_bindings import BF16, FP16


def test_l2_closed_form(oracle):
    # test/doctest_losses.cpp:46-51: value = (p-t)^2/N, grad = loss_scale*2*(p-t)/N
    n = 64 * 8
    pred = np.full(n, 0.5, np.float32)
    targ = np.full(n, 0.125, np.float32)
    values, grads = oracle.l2_loss(FP16, pred, targ, 4.0)
    assert np.allclose(values, 0.375 ** 2 / n)
    assert np.allclose(grads, 4.0 * 2 * 0.375 / n, rtol=1e-3)
    assert abs(values.sum() - 0.375 ** 2) < 1e-6


def test_l2_matches_torch_mse(oracle):
    rng = np.random.default_rng(0)
    p = oracle.round(rng.standard_normal(4096), BF16)
    t = rng.uniform(0, 1, 4096).astype(np.float32)
    values, grads = oracle.l2_loss(BF16, p, t, 1.0)
    tp = torch.tensor(p, requires_grad=True)
    loss = torch.nn.functional.mse_loss(tp, torch.tensor(t))
    loss.backward()
    assert abs(values.sum() - loss.item()) < 1e-6
    assert np.allclose(grads, tp.grad.numpy(), rtol=2 ** -7, atol=1e-12)


def test_adam_matches_torch(oracle):
    rng = np.random.default_rng(1)
    n = 1000
    p0 = rng.standard_normal(n).astype(np.float32)
    tp = torch.nn.Parameter(torch.tensor(p0.copy()))
    opt = torch.optim.Adam([tp], lr=1e-3, betas=(0.9, 0.99), eps=1e-15)
    p, m, v = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for step in range(1, 6):
        g = rng.standard_normal(n).astype(np.float32) * 0.1
        tp.grad = torch.tensor(g)
        opt.step()
        p, m, v = oracle.adam_step(p, m, v, g, step, 1e-3, 0.9, 0.99, 1e-15)
        assert np.allclose(p, tp.detach().numpy(), rtol=1e-6, atol=1e-7)
