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


def test_fill_uniform_generator(oracle):
    """The seeded uniform fill that stands in for the reference's unseeded / closed-source initialisers. Its bit source is
    splitmix64: pinned by the first outputs of Vigna's public-domain splitmix64.c for the seed 1234567 and by an
    independent big-integer evaluation; the floats by range, mean, variance and the exact 24-bit construction."""
    vigna = [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431, 16408922859458223821]
    assert [oracle.splitmix64(1234567, i) for i in range(5)] == vigna
    mask = (1 << 64) - 1

    def mix(seed, i):
        z = (seed + (i + 1) * 0x9E3779B97F4A7C15) & mask
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        return z ^ (z >> 31)

    assert all(oracle.splitmix64(s, i) == mix(s, i) for s in (0, 777, mask) for i in (0, 1, 2 ** 40, mask - 1))
    from oracle_bindings import FP32
    n = 1 << 18
    v = oracle.fill_uniform(n, -1e-4, 1e-4, 777, 0, FP32)
    assert v.min() >= -1e-4 and v.max() < 1e-4
    assert abs(v.mean()) < 3 * 2e-4 / np.sqrt(12 * n) and abs(v.var() / ((2e-4) ** 2 / 12) - 1) < 0.02
    # element i depends on (seed, first_index + i) only
    assert np.array_equal(oracle.fill_uniform(100, -1e-4, 1e-4, 777, 1000, FP32), v[1000:1100])
    u = oracle.fill_uniform(64, 0.0, 1.0, 5, 0, FP32)
    assert np.array_equal(u, np.array([(mix(5, i) >> 40) / 2.0 ** 24 for i in range(64)], np.float32))
    h = oracle.fill_uniform(4096, -0.25, 0.25, 9, 0, BF16)
    assert np.array_equal(h, oracle.round(oracle.fill_uniform(4096, -0.25, 0.25, 9, 0, FP32), BF16))
