"""tnn_mlp_train_step_l2_static: the training step whose scratch memory is a fixed device array inside the
library (for callers that cannot allocate). Its results must equal tnn_mlp_train_step_l2's bit for bit, on
calls in a row that share the array, the second with a smaller input. Collected last on purpose (file name)."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from tolerances import BF16, FP16  # noqa: E402


def _case(tnn, oracle, dtype, W, n_hidden, M, seed):
    import torch
    rng = np.random.default_rng(seed)
    n_mats = n_hidden + 1
    lim = np.sqrt(6.0 / (2 * W))
    w = oracle.round(rng.uniform(-lim, lim, (n_mats, W, W)), dtype)
    x = oracle.round(rng.uniform(-1, 1, (M, W)), dtype)
    targets = rng.uniform(0, 1, (M, W)).astype(np.float32)
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    _, pf, pb = tnn.prepare(desc, w)
    return desc, pf, pb, tnn.dev_tensor(x, dtype), torch.from_numpy(targets).to(tnn.dev), w


def _static_step(tnn, desc, pf, pb, xt, tt, loss_scale, dw_fp32=True):
    import torch
    from tiny_dpcpp_nn import _lib
    from tiny_dpcpp_nn.cabi import ptr
    M, W = xt.shape
    n_mats = desc.n_hidden_layers + 1
    y = torch.full_like(xt, float("nan"))
    dX = torch.full_like(xt, float("nan"))
    loss = torch.full((1,), float("nan"), dtype=torch.float32, device=tnn.dev)
    dW = torch.full((n_mats, W, W), float("nan"), dtype=torch.float32 if dw_fp32 else xt.dtype, device=tnn.dev)
    _lib.check(tnn.lib.tnn_mlp_train_step_l2_static(ctypes.byref(desc), ptr(pf), ptr(pb), ptr(xt), ptr(tt), loss_scale, ptr(y), ptr(loss),
                                                    ptr(dW), int(dw_fp32), ptr(dX), M, tnn.stream()))
    return y, loss, dW, dX


def _same(a, b):
    import torch
    return all(torch.equal(p.view(torch.uint8), q.view(torch.uint8)) for p, q in zip(a, b))


def test_static_scratch_step_equals_the_workspace_step(tnn, oracle):
    import torch
    # two calls in a row on the shared array, the second with fewer rows (fewer workgroups, so stale partials of the
    # first call lie behind the ones it writes), then a different shape and type, then the first again
    shapes = ((BF16, 64, 4, 1 << 16, 1), (BF16, 64, 4, 1000 * 8, 2), (FP16, 32, 2, 4096 + 8, 3), (BF16, 64, 4, 1 << 16, 1))
    cases = [_case(tnn, oracle, dtype, W, n_hidden, M, seed) for dtype, W, n_hidden, M, seed in shapes]
    got = [_static_step(tnn, desc, pf, pb, xt, tt, 4.0) for desc, pf, pb, xt, tt, _ in cases]  # back to back on the shared array
    torch.cuda.synchronize()
    for (desc, pf, pb, xt, tt, _), g, (_, W, _, M, _) in zip(cases, got, shapes):
        want = tnn.train_step_l2(desc, pf, pb, xt, tt, 4.0)
        torch.cuda.synchronize()
        assert not any(torch.isnan(t.float()).any().item() for t in g)
        assert _same(g, want), f"static-scratch step differs from the workspace step (W={W}, M={M})"
    # and against the oracle directly, so that the pair cannot be wrong together
    desc, pf, pb, xt, tt, w = _case(tnn, oracle, BF16, 64, 2, 2048, 7)
    y, loss, dW, dX = _static_step(tnn, desc, pf, pb, xt, tt, 1.0)
    from tolerances import assert_propagated
    interm = oracle.mlp_forward_T(BF16, 64, 3, "relu", "none", w, tnn.host(xt))
    assert_propagated(tnn.host(y), interm[-1], BF16, "static step: output")
    _, grads = oracle.l2_loss(BF16, tnn.host(y), tnn.host(tt), 1.0)
    _, rdW, _ = oracle.mlp_backward_T(BF16, 64, 3, "relu", "none", w, interm, grads, round_dw=False)
    assert_propagated(tnn.host(dW), rdW, BF16, "static step: dW", scale=float(np.abs(rdW).max()))


def test_static_scratch_rejects_what_does_not_fit(tnn):
    from tiny_dpcpp_nn import _lib
    lib = tnn.lib
    cap = lib.tnn_mlp_train_step_l2_static_max_bytes()
    assert cap == 21 << 20
    # every shape with the fused kernel fits whatever the batch size
    for W, L in ((64, 4), (32, 5), (16, 5), (64, 1)):
        d = tnn.mlp_desc(BF16, W, L, "relu", "none")
        assert 0 < lib.tnn_mlp_train_step_workspace_bytes(ctypes.byref(d), 1 << 22) <= cap
    # width 128 stages activations in its workspace: too large at this batch size, and said so before anything is launched
    wide = tnn.mlp_desc(FP16, 128, 8, "relu", "none")
    rc = lib.tnn_mlp_train_step_l2_static(ctypes.byref(wide), None, None, None, None, 1.0, None, None, None, 1, None, 1 << 16, None)
    assert rc == _lib.TNN_ERR_WORKSPACE and b"static buffer holds" in lib.tnn_last_error()
