"""Parity of the fused MLP kernels (through the C ABI) with the oracle, on seeded inputs."""
import ctypes

import numpy as np
import pytest

from tolerances import BF16, FP16, FP32, PROPAGATED, assert_close, assert_propagated, max_norm_rel

pytestmark = pytest.mark.gpu

ACTS = ["none", "relu", "sigmoid"]


def xavier(W, n_mats, seed):
    rng = np.random.default_rng(seed)
    lim = np.sqrt(6.0 / (2 * W))
    return rng.uniform(-lim, lim, (n_mats, W, W))


def make_case(oracle, dtype, W, n_mats, M, seed=0):
    rng = np.random.default_rng(1234 + seed)
    w = oracle.round(xavier(W, n_mats, 42 + seed), dtype)
    x = oracle.round(rng.uniform(-1, 1, (M, W)), dtype)
    return w, x


def test_prepare_and_layout_kernels_bit_exact(tnn, oracle):
    for dtype in (BF16, FP16):
        for W in (16, 64):
            n_mats = 3
            w = oracle.round(np.random.default_rng(W).standard_normal(n_mats * W * W), dtype)
            unp = tnn.dev_tensor(w, dtype)
            packed = tnn.pack(dtype, W, n_mats, unp)
            assert np.array_equal(tnn.host(packed), oracle.pack_weights(w, n_mats, W))
            import torch
            from tiny_dpcpp_nn import _lib
            from gpu_harness import ptr
            back = torch.empty_like(unp)
            _lib.check(tnn.lib.tnn_unpack_weights(dtype, W, n_mats, ptr(packed), ptr(back), tnn.stream()))
            assert np.array_equal(tnn.host(back), w)
            pt = torch.empty_like(unp)
            _lib.check(tnn.lib.tnn_packed_transpose(dtype, W, n_mats, ptr(packed), ptr(pt), tnn.stream()))
            exp = np.concatenate([oracle.packed_transpose(oracle.pack_weights(w[m * W * W:(m + 1) * W * W], 1, W), W) for m in range(n_mats)])
            assert np.array_equal(tnn.host(pt), exp)
            pat = torch.empty_like(unp)
            _lib.check(tnn.lib.tnn_pack_and_transpose(dtype, W, n_mats, ptr(unp), ptr(pat), tnn.stream()))
            exp = np.concatenate([oracle.pack_and_transpose(w[m * W * W:(m + 1) * W * W], W) for m in range(n_mats)])
            assert np.array_equal(tnn.host(pat), exp)
            desc = tnn.mlp_desc(dtype, W, n_mats - 1, "relu", "none")
            for (n_in, n_out, bias) in ((3, 5, True), (3, 5, False), (16, W, True)):
                z = packed.clone()
                _lib.check(tnn.lib.tnn_zero_weights_padding(ctypes.byref(desc), ptr(z), n_in, n_out, int(bias), tnn.stream()))
                assert np.array_equal(tnn.host(z), oracle.zero_weights_padding(oracle.pack_weights(w, n_mats, W), n_mats, W, n_in, n_out, bias))
                # the one-launch route of a module's push: the same four copies as cast + zero padding + packed transpose + prepare
                zt = torch.empty_like(z)
                _lib.check(tnn.lib.tnn_packed_transpose(dtype, W, n_mats, ptr(z), ptr(zt), tnn.stream()))
                pf, pb = tnn.prepare_packed(desc, z)
                for src in (packed, packed.float()):
                    outs = [torch.full_like(t, float("nan")) for t in (z, zt, pf, pb)]
                    _lib.check(tnn.lib.tnn_mlp_set_packed_weights(ctypes.byref(desc), ptr(src), FP32 if src.dtype == torch.float32 else dtype, n_in, n_out,
                                                                  int(bias), ptr(outs[0]), ptr(outs[1]), ptr(outs[2]), ptr(outs[3]), tnn.stream()))
                    for got, want in zip(outs, (z, zt, pf, pb)):
                        assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("dtype", [BF16, FP16])
@pytest.mark.parametrize("W,n_hidden", [(16, 2), (32, 4), (64, 4), (128, 8), (64, 1), (128, 2)])
def test_inference_and_forward_parity(tnn, oracle, dtype, W, n_hidden):
    n_mats = n_hidden + 1
    M = 8 * 37  # a multiple of 8 that is not a multiple of the 32-row tile
    w, x = make_case(oracle, dtype, W, n_mats, M, seed=W + n_hidden)
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    _, pf, _ = tnn.prepare(desc, w)
    xt = tnn.dev_tensor(x, dtype)
    ref = oracle.mlp_forward_T(dtype, W, n_mats, "relu", "none", w, x)
    y = tnn.host(tnn.inference(desc, pf, xt))
    assert_propagated(y, ref[-1], dtype, "inference output")
    interm = tnn.host(tnn.forward(desc, pf, xt))
    assert np.array_equal(interm[0], x)
    for l in range(1, n_mats + 1):
        assert_propagated(interm[l], ref[l], dtype, f"interm_fwd[{l}]")
        # one layer at a time on identical inputs: every element inside the bar
        one = oracle.mlp_forward_T(dtype, W, 1, "none", "relu" if l < n_mats else "none", w[l - 1], interm[l - 1], store_interm=False)
        assert_close(interm[l], one, dtype, f"layer {l} on the GPU's own input")
    assert np.array_equal(interm[-1], y)
    # the reference's own bar against the double-precision oracle (test/doctest_swiftnet.cpp:517-576)
    ref64 = oracle.mlp_forward_f64(W, n_mats, "relu", "none", w, x)
    for l in range(1, n_mats + 1):
        assert max_norm_rel(interm[l], ref64[l]) < 1e-2


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("out_act", ACTS)
def test_activation_pairs_forward_backward(tnn, oracle, act, out_act):
    # the 3 x 3 activation matrix of test/doctest_swiftnet.cpp:931-966, both dtypes
    for dtype, ls in ((BF16, 1.0), (FP16, 128.0)):
        W, n_hidden, M = 64, 3, 136
        n_mats = n_hidden + 1
        w, x = make_case(oracle, dtype, W, n_mats, M, seed=7)
        g = oracle.round(np.random.default_rng(5).uniform(-1, 1, (M, W)) * ls / M, dtype)
        desc = tnn.mlp_desc(dtype, W, n_hidden, act, out_act)
        _, pf, pb = tnn.prepare(desc, w)
        interm_t = tnn.forward(desc, pf, tnn.dev_tensor(x, dtype))
        interm = tnn.host(interm_t)
        ref = oracle.mlp_forward_T(dtype, W, n_mats, act, out_act, w, x)
        for l in range(1, n_mats + 1):
            assert_propagated(interm[l], ref[l], dtype, f"{act}/{out_act} interm_fwd[{l}]")
            one = oracle.mlp_forward_T(dtype, W, 1, "none", act if l < n_mats else out_act, w[l - 1], interm[l - 1], store_interm=False)
            assert_close(interm[l], one, dtype, f"{act}/{out_act} layer {l} on the GPU's own input")
        # backward on the activations the GPU forward produced (the oracle gets the same ones)
        ib, dW, dX = tnn.backward(desc, pb, tnn.dev_tensor(g, dtype), interm_t)
        rib, rdW, rdX = oracle.mlp_backward_T(dtype, W, n_mats, act, out_act, w, interm, g)
        gs = ls / M
        for l in range(n_mats):
            assert_propagated(tnn.host(ib[l]), rib[l], dtype, f"{act}/{out_act} delta[{l}]", scale=gs)
        assert_propagated(tnn.host(dX), rdX, dtype, "dL/dx", scale=gs)
        assert_propagated(tnn.host(dW), rdW, dtype, "dW", scale=ls)
        for l in range(n_mats):
            assert max_norm_rel(tnn.host(dW[l]), rdW[l]) < 1e-2


@pytest.mark.parametrize("dtype", [BF16, FP16])
@pytest.mark.parametrize("W,n_hidden", [(16, 2), (32, 4), (128, 8), (64, 4), (128, 3)])
def test_backward_parity_widths(tnn, oracle, dtype, W, n_hidden):
    n_mats = n_hidden + 1
    M = 8 * 45
    ls = 128.0 if dtype == FP16 else 1.0
    w, x = make_case(oracle, dtype, W, n_mats, M, seed=3)
    g = oracle.round(np.random.default_rng(6).uniform(-1, 1, (M, W)) * ls / M, dtype)
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    _, pf, pb = tnn.prepare(desc, w)
    interm_t = tnn.forward(desc, pf, tnn.dev_tensor(x, dtype))
    interm = tnn.host(interm_t)
    rib, rdW, rdX = oracle.mlp_backward_T(dtype, W, n_mats, "relu", "none", w, interm, g, round_dw=False)
    # deltas kept on chip / in the workspace, fp32 weight gradients, no dL/dx
    ib, dW, dX = tnn.backward(desc, pb, tnn.dev_tensor(g, dtype), interm_t, want_interm=False, want_dx=False, dw_fp32=True)
    assert ib is None and dX is None
    assert_propagated(tnn.host(dW), rdW, dtype, "dW fp32", scale=ls)
    # and the reference-shaped call
    ib, dW2, dX = tnn.backward(desc, pb, tnn.dev_tensor(g, dtype), interm_t)
    for l in range(n_mats):
        assert_propagated(tnn.host(ib[l]), rib[l], dtype, f"delta[{l}]", scale=ls / M)
    assert_propagated(tnn.host(dX), rdX, dtype, "dL/dx", scale=ls / M)
    assert_propagated(tnn.host(dW2), oracle.round(rdW, dtype), dtype, "dW", scale=ls)
    # dW given the deltas the GPU itself produced is a plain product: strict bar, every element
    gib = tnn.host(ib)
    for l in range(n_mats):
        exact = gib[l].astype(np.float64).T @ interm[l].astype(np.float64)
        assert_close(tnn.host(dW[l]), exact, dtype, f"dW[{l}] from the GPU's own deltas", scale=ls)
    # against the double oracle fed the same activations (test/doctest_swiftnet.cpp:99-233)
    d64, dW64, dX64 = oracle.mlp_backward_f64(W, n_mats, "relu", "none", w, np.concatenate([x[None], interm[1:]]), g)
    for l in range(n_mats):
        assert max_norm_rel(tnn.host(dW2[l]), dW64[l]) < 1e-2
        assert max_norm_rel(tnn.host(ib[l]), d64[l]) < 1e-2
    assert max_norm_rel(tnn.host(dX), dX64) < 1e-2


def test_closed_forms(tnn, oracle):
    # test/doctest_swiftnet.cpp:44-51,79-96 : constant weights 0.01 with padded input / output
    dtype, W, n_hidden, M = BF16, 64, 2, 16
    n_mats = n_hidden + 1
    n_in, n_out = 7, 5
    w = np.full((n_mats, W, W), 0.01)
    w[0, n_in:, :] = 0
    w[-1, :, n_out:] = 0
    w = oracle.round(w, dtype)
    x = np.zeros((M, W)); x[:, :n_in] = 1.0
    desc = tnn.mlp_desc(dtype, W, n_hidden, "none", "none")
    _, pf, pb = tnn.prepare(desc, w)
    interm = tnn.host(tnn.forward(desc, pf, tnn.dev_tensor(x, dtype)))
    c = float(oracle.round(np.float32([0.01]), dtype)[0])
    assert np.allclose(interm[1], c * n_in, rtol=1e-2)
    assert np.allclose(interm[2], c * n_in * W * c, rtol=1e-2)
    assert np.allclose(interm[3][:, :n_out], c * n_in * W * c * W * c, rtol=2e-2)
    assert np.all(interm[3][:, n_out:] == 0)
    # benchmarks/benchmark_inference.h:47-48,71 and benchmark_training.h:48-59,90-96 (weights 1/W)
    for W in (16, 32, 64, 128):
        n_hidden, B = 4, 64
        n_mats = n_hidden + 1
        w = np.full((n_mats, W, W), 1.0 / W)
        v = float(oracle.round(np.float32([np.sqrt(1.0 / B)]), dtype)[0])
        desc = tnn.mlp_desc(dtype, W, n_hidden, "none", "none")
        _, pf, pb = tnn.prepare(desc, w)
        xt = tnn.dev_tensor(np.full((B, W), v), dtype)
        interm_t = tnn.forward(desc, pf, xt)
        assert np.all(tnn.host(interm_t) == v)
        ib, dW, dX = tnn.backward(desc, pb, xt, interm_t, dw_fp32=True)
        assert np.all(tnn.host(ib) == v) and np.all(tnn.host(dX) == v)
        assert np.allclose(tnn.host(dW), B * v * v, rtol=1e-6)


def test_argument_checks(tnn):
    """Error behaviour of the reference's checks, as status codes (no GPU work is launched)."""
    import torch
    from tiny_dpcpp_nn import _lib
    from gpu_harness import ptr
    desc = tnn.mlp_desc(BF16, 64, 2, "relu", "none")
    buf = torch.zeros(64 * 64 * 8, dtype=torch.bfloat16, device=tnn.dev)
    # include/network/SwiftNetMLP.h:293-300 / test/doctest_swiftnet.cpp:891-905: batch 1 and 13 are rejected, 8 is fine
    for M in (1, 13, 0):
        assert tnn.lib.tnn_mlp_inference(ctypes.byref(desc), ptr(buf), ptr(buf), ptr(buf), M, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    for bad in (tnn.mlp_desc(BF16, 48, 2, "relu", "none"), tnn.mlp_desc(BF16, 64, 0, "relu", "none")):
        assert tnn.lib.tnn_mlp_inference(ctypes.byref(bad), ptr(buf), ptr(buf), ptr(buf), 8, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    bad = tnn.mlp_desc(BF16, 64, 2, _lib.ACT_TANH, "none")
    assert tnn.lib.tnn_mlp_inference(ctypes.byref(bad), ptr(buf), ptr(buf), ptr(buf), 8, None) == _lib.TNN_ERR_UNSUPPORTED
    assert tnn.lib.tnn_mlp_inference(ctypes.byref(desc), None, ptr(buf), ptr(buf), 8, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert tnn.lib.tnn_mlp_backward(ctypes.byref(desc), ptr(buf), ptr(buf), ptr(buf), None, ptr(buf), 0, None, 8, ptr(buf), 16, None) == _lib.TNN_ERR_WORKSPACE
    assert b"workspace" in tnn.lib.tnn_last_error()


@pytest.mark.parametrize("dtype,W,n_hidden,M", [
    (FP16, 128, 2, (1 << 16) + 24),  # width 128, few matrices, activations stored: the route that streams the matrices through LDS
    (BF16, 64, 4, (1 << 20) + 8),    # 805 MB of activations: whole-row stores with the streaming hint
    (FP16, 32, 4, (1 << 18) + 40),   # two rows per 128-byte line
    (FP16, 16, 2, (1 << 18) + 8),    # four rows per line
])
def test_forward_store_routes_at_large_batches(tnn, oracle, dtype, W, n_hidden, M):
    """The row stores of forward and inference take different routes with the batch size and the shape (plain, through a
    staged tile, with or without the streaming hint). Rows are independent, so the first and the last 96 rows of a large,
    ragged batch are compared with the oracle, matrix by matrix, and the two calls with each other over the whole batch."""
    import torch
    from gpu_harness import TORCH_DT
    n_mats = n_hidden + 1
    w = oracle.round(xavier(W, n_mats, 5), dtype)
    gen = torch.Generator(device=tnn.dev).manual_seed(9)
    xt = (torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1).to(TORCH_DT[dtype])
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    _, pf, _ = tnn.prepare(desc, w)
    interm_t = tnn.forward(desc, pf, xt)  # pre-filled with NaN by the harness
    y_t = tnn.inference(desc, pf, xt)
    assert not torch.isnan(interm_t).any(), "rows left unwritten"
    assert torch.equal(interm_t[n_mats], y_t), "forward and inference disagree"
    assert torch.equal(interm_t[0], xt), "interm_fwd[0] is not the input"
    for rows in (slice(0, 96), slice(M - 96, M)):
        ref = oracle.mlp_forward_T(dtype, W, n_mats, "relu", "none", w, tnn.host(xt[rows]))
        for l in range(1, n_mats + 1):
            assert_propagated(tnn.host(interm_t[l][rows]), ref[l], dtype, f"interm_fwd[{l}] rows {rows}")


def test_matrices_beyond_two_gib(tnn, oracle):
    """A matrix of more than 2 GiB does not fit the 32-bit offsets of the range-checked row stores: forward, inference and
    backward then take the plain routes. 2^24 + 8 rows of width 64 (2.1 GB per matrix), one hidden layer."""
    import torch
    from gpu_harness import TORCH_DT
    dtype, W, n_hidden, M = BF16, 64, 1, (1 << 24) + 8
    n_mats = n_hidden + 1
    w = oracle.round(xavier(W, n_mats, 11), dtype)
    gen = torch.Generator(device=tnn.dev).manual_seed(12)
    xt = (torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1).to(TORCH_DT[dtype])
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    _, pf, pb = tnn.prepare(desc, w)
    interm_t = tnn.forward(desc, pf, xt)
    y_t = tnn.inference(desc, pf, xt)
    assert torch.equal(interm_t[n_mats], y_t) and torch.equal(interm_t[0], xt)
    assert not torch.isnan(interm_t[1]).any()
    gt = ((torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1) / M).to(TORCH_DT[dtype])
    ib, dW, dX = tnn.backward(desc, pb, gt, interm_t, dw_fp32=True)
    assert not torch.isnan(ib).any() and not torch.isnan(dX).any() and not torch.isnan(dW).any()
    for rows in (slice(0, 96), slice(M - 96, M)):
        ref = oracle.mlp_forward_T(dtype, W, n_mats, "relu", "none", w, tnn.host(xt[rows]))
        for l in range(1, n_mats + 1):
            assert_propagated(tnn.host(interm_t[l][rows]), ref[l], dtype, f"interm_fwd[{l}] rows {rows}")
        rib, _, rdX = oracle.mlp_backward_T(dtype, W, n_mats, "relu", "none", w, tnn.host(interm_t[:, rows]), tnn.host(gt[rows]), round_dw=False)
        for l in range(n_mats):
            assert_propagated(tnn.host(ib[l][rows]), rib[l], dtype, f"delta[{l}] rows {rows}", scale=1.0 / M)
        assert_propagated(tnn.host(dX[rows]), rdX, dtype, f"dL/dx rows {rows}", scale=1.0 / M)
    for l in range(n_mats):
        exact = torch.zeros((W, W), dtype=torch.float64, device=tnn.dev)
        for r0 in range(0, M, 1 << 22):  # in pieces: the fp64 copies of whole matrices would take 17 GB each
            exact += ib[l][r0:r0 + (1 << 22)].double().T @ interm_t[l][r0:r0 + (1 << 22)].double()
        assert_close(tnn.host(dW[l]), exact.cpu().numpy(), dtype, f"dW[{l}] from the GPU's own deltas")


@pytest.mark.parametrize("dtype,W,n_hidden,M", [(BF16, 64, 4, (1 << 18) + 40), (FP16, 32, 2, (1 << 18) + 8), (FP16, 16, 2, (1 << 18) + 24)])
def test_backward_store_route_at_large_batch(tnn, oracle, dtype, W, n_hidden, M):
    """The fused backward writes its deltas and dL/dx as whole rows from staged tiles, through range-checked buffer stores.
    Large ragged batch: nothing left unwritten, first and last rows against the oracle, and the weight gradients against
    the product of the deltas and activations the GPU itself holds (fp64 on the device)."""
    import torch
    from gpu_harness import TORCH_DT
    n_mats = n_hidden + 1
    ls = 128.0 if dtype == FP16 else 1.0
    w = oracle.round(xavier(W, n_mats, 8), dtype)
    gen = torch.Generator(device=tnn.dev).manual_seed(10)
    xt = (torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1).to(TORCH_DT[dtype])
    gt = ((torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1) * (ls / M)).to(TORCH_DT[dtype])
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    _, pf, pb = tnn.prepare(desc, w)
    interm_t = tnn.forward(desc, pf, xt)
    ib, dW, dX = tnn.backward(desc, pb, gt, interm_t, dw_fp32=True)  # outputs pre-filled with NaN by the harness
    assert not torch.isnan(ib).any() and not torch.isnan(dX).any() and not torch.isnan(dW).any()
    for rows in (slice(0, 96), slice(M - 96, M)):
        rib, _, rdX = oracle.mlp_backward_T(dtype, W, n_mats, "relu", "none", w, tnn.host(interm_t[:, rows]), tnn.host(gt[rows]), round_dw=False)
        for l in range(n_mats):
            assert_propagated(tnn.host(ib[l][rows]), rib[l], dtype, f"delta[{l}] rows {rows}", scale=ls / M)
        assert_propagated(tnn.host(dX[rows]), rdX, dtype, f"dL/dx rows {rows}", scale=ls / M)
    for l in range(n_mats):
        exact = (ib[l].double().T @ interm_t[l].double()).cpu().numpy()
        assert_close(tnn.host(dW[l]), exact, dtype, f"dW[{l}] from the GPU's own deltas", scale=ls)


def test_baseline_config_1_full_size(tnn, oracle):
    """BASELINE config 1: w64, 4 hidden layers, bf16, ReLU / linear, batch 2^17, compared row for row."""
    dtype, W, n_hidden, M = BF16, 64, 4, 1 << 17
    n_mats = n_hidden + 1
    w, x = make_case(oracle, dtype, W, n_mats, M)
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    _, pf, _ = tnn.prepare(desc, w)
    y = tnn.host(tnn.inference(desc, pf, tnn.dev_tensor(x, dtype)))
    ref = oracle.mlp_forward_T(dtype, W, n_mats, "relu", "none", w, x, store_interm=False)
    assert_propagated(y, ref, dtype, "config 1 output")
    # against the double-precision oracle, which never rounds between layers, the reference's own bar
    # applies: max-norm relative difference 1e-2 (test/doctest_swiftnet.cpp:183,225-227)
    ref64 = oracle.mlp_forward_f64(W, n_mats, "relu", "none", w, x)[-1]
    assert max_norm_rel(y, ref64) < 1e-2


def test_baseline_config_2_training_step(tnn, oracle):
    """BASELINE config 2: one training step (forward, L2 against U[0,1) targets, backward with dW, Adam)
    at batch 2^18; every stage checked against the oracle."""
    import torch
    dtype, W, n_hidden, M = BF16, 64, 4, 1 << 18
    n_mats = n_hidden + 1
    w, x = make_case(oracle, dtype, W, n_mats, M)
    rng = np.random.default_rng(99)
    targets = rng.uniform(0, 1, (M, W)).astype(np.float32)
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    packed, pf, pb = tnn.prepare(desc, w)
    xt, tt = tnn.dev_tensor(x, dtype), torch.from_numpy(targets).to(tnn.dev)
    y, loss, dW, dX = tnn.train_step_l2(desc, pf, pb, xt, tt, 1.0)
    y = tnn.host(y)
    interm = oracle.mlp_forward_T(dtype, W, n_mats, "relu", "none", w, x)
    assert_propagated(y, interm[-1], dtype, "output")
    values, grads = oracle.l2_loss(dtype, y, targets, 1.0)
    assert abs(float(loss.item()) - float(values.astype(np.float64).sum())) < 1e-4 * float(values.astype(np.float64).sum())
    # oracle backward on the oracle's own forward; ReLU masks of the (rare) activations that round
    # differently move single rows, which a batch-summed dW tolerates at the stated bar
    rib, rdW, rdX = oracle.mlp_backward_T(dtype, W, n_mats, "relu", "none", w, interm, grads, round_dw=False)
    dWh = tnn.host(dW)
    for l in range(n_mats):
        assert max_norm_rel(dWh[l], rdW[l]) < 1e-2
    assert_propagated(dWh, rdW, dtype, "dW", scale=float(np.abs(rdW).max()))
    # Adam (torch semantics) on fp32 masters kept in the packed layout
    master = tnn.host(packed).astype(np.float32)
    gp = np.concatenate([oracle.pack_and_transpose(dWh[l].ravel(), W) for l in range(n_mats)])
    from gpu_harness import ptr
    from tiny_dpcpp_nn import _lib
    dWp = torch.empty(n_mats * W * W, dtype=torch.float32, device=tnn.dev)
    _lib.check(tnn.lib.tnn_pack_and_transpose(2, W, n_mats, ptr(dW), ptr(dWp), tnn.stream()))
    assert np.array_equal(tnn.host(dWp), gp)
    p = torch.from_numpy(master.copy()).to(tnn.dev)
    m = torch.zeros_like(p)
    v = torch.zeros_like(p)
    pT = torch.empty(p.shape, dtype=torch.bfloat16, device=tnn.dev)
    tnn.adam_step(p, m, v, dWp, 2, 1.0, 1, 1e-3, 0.9, 0.99, 1e-15, pT, BF16)
    rp, rm, rv = oracle.adam_step(master, np.zeros_like(master), np.zeros_like(master), gp, 1, 1e-3, 0.9, 0.99, 1e-15)
    assert np.allclose(tnn.host(p), rp, rtol=1e-6, atol=1e-7)
    assert np.allclose(tnn.host(m), rm, rtol=1e-6, atol=1e-9) and np.allclose(tnn.host(v), rv, rtol=1e-6, atol=1e-12)
    assert np.array_equal(tnn.host(pT), oracle.round(tnn.host(p), BF16))
    # the one-call entry point (the one the benchmark times): same step with Adam applied inside the gradient reduction
    p2 = torch.from_numpy(master.copy()).to(tnn.dev)
    m2, v2 = torch.zeros_like(p2), torch.zeros_like(p2)
    pT2 = torch.empty(p2.shape, dtype=torch.bfloat16, device=tnn.dev)
    pf2, pb2 = pf.clone(), pb.clone()
    y2, dX2 = torch.empty_like(xt), torch.empty_like(xt)
    loss2 = torch.full((1,), float("nan"), device=tnn.dev)
    ws_bytes = tnn.lib.tnn_mlp_train_step_workspace_bytes(ctypes.byref(desc), M)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=tnn.dev)
    _lib.check(tnn.lib.tnn_mlp_train_step_l2_adam(ctypes.byref(desc), ptr(pf2), ptr(pb2), ptr(xt), ptr(tt), 1.0, ptr(y2), ptr(loss2), ptr(p2),
                                                  ptr(m2), ptr(v2), 1, 1e-3, 0.9, 0.99, 1e-15, ptr(pT2), ptr(dX2), M, ptr(ws), ws_bytes, None,
                                                  tnn.stream()))
    assert_propagated(tnn.host(y2), interm[-1], dtype, "output of the one-call step")
    assert abs(float(loss2.item()) - float(values.astype(np.float64).sum())) < 1e-4 * float(values.astype(np.float64).sum())
    # dL/dx: bit-equal to the step without Adam; against the oracle's backward over the oracle's own forward the elementwise
    # bar holds, while single rows whose ReLU mask flipped on a rounding boundary are outside any max-norm bound
    assert torch.equal(dX2.view(torch.int16), dX.view(torch.int16))
    from tolerances import PROPAGATED
    assert_close(tnn.host(dX2), rdX, dtype, "dL/dx of the one-call step", scale=1.0 / M, frac_ok=PROPAGATED)
    assert np.allclose(tnn.host(p2), rp, rtol=1e-6, atol=1e-7)
    assert np.allclose(tnn.host(m2), rm, rtol=1e-6, atol=1e-9) and np.allclose(tnn.host(v2), rv, rtol=1e-6, atol=1e-12)
    assert np.array_equal(tnn.host(pT2), oracle.round(tnn.host(p2), BF16))
    # the weights it re-staged for the next step are the rounded masters in both operand orders
    wf_ref, wb_ref = tnn.prepare_packed(desc, p2, src_is_fp32=True)
    assert torch.equal(pf2.view(torch.int16), wf_ref.view(torch.int16)) and torch.equal(pb2.view(torch.int16), wb_ref.view(torch.int16))


def test_linearity_property_full_size(tnn, oracle):
    """Size-independent property at batch 2^20 (config 3 size): with no activation the network is
    linear, so f(2x) == 2 f(x) exactly in binary floating point, and rows are independent of the
    batch they travel in."""
    import torch
    dtype, W, n_hidden, M = FP16, 32, 4, 1 << 20
    w = oracle.round(xavier(W, n_hidden + 1, 1), dtype)
    desc = tnn.mlp_desc(dtype, W, n_hidden, "none", "none")
    _, pf, _ = tnn.prepare(desc, w)
    x = torch.rand((M, W), device=tnn.dev, generator=torch.Generator(device=tnn.dev).manual_seed(3)).mul_(2).sub_(1).to(torch.float16)
    y1 = tnn.inference(desc, pf, x)
    y2 = tnn.inference(desc, pf, x * 2)
    # exact in binary floating point except where an activation on the way is an fp16 denormal (their
    # fixed quantum does not scale with the input): nearly every row is bit-identical, all are inside the bar
    exact = (y2 == y1 * 2).all(dim=1)
    assert float(exact.float().mean()) > 0.995  # about 0.13% of the rows hold an output below 2^-14
    assert_close(y2.float().cpu().numpy(), (y1.float() * 2).cpu().numpy(), FP16, "f(2x) vs 2 f(x)")
    ys = tnn.inference(desc, pf, x[1000:1000 + 4096].contiguous())
    assert torch.equal(ys, y1[1000:1000 + 4096])


@pytest.mark.parametrize("dtype", [BF16, FP16])
@pytest.mark.parametrize("W,n_hidden,act,out_act", [(64, 4, "relu", "none"), (64, 2, "relu", "none"), (64, 1, "sigmoid", "sigmoid"),
                                                    (32, 4, "relu", "relu"), (32, 5, "none", "none"), (16, 2, "relu", "none"),
                                                    (16, 1, "sigmoid", "none"), (64, 3, "none", "sigmoid"), (128, 2, "relu", "none"),
                                                    (64, 6, "relu", "none"), (128, 3, "relu", "sigmoid"), (128, 1, "sigmoid", "relu")])
def test_train_step_single_call(tnn, oracle, dtype, W, n_hidden, act, out_act):
    """tnn_mlp_train_step_l2 (one kernel for widths <= 64 and <= 4-5 hidden layers, separate kernels over
    workspace matrices otherwise) against forward + L2 + backward called one by one, and against the oracle."""
    import torch
    n_mats = n_hidden + 1
    M = 8 * 331  # several rounds of partially filled workgroups, last tile ragged
    ls = 128.0 if dtype == FP16 else 1.0
    w, x = make_case(oracle, dtype, W, n_mats, M, seed=n_hidden)
    targets = np.random.default_rng(77).uniform(0, 1, (M, W)).astype(np.float32)
    desc = tnn.mlp_desc(dtype, W, n_hidden, act, out_act)
    _, pf, pb = tnn.prepare(desc, w)
    xt, tt = tnn.dev_tensor(x, dtype), torch.from_numpy(targets).to(tnn.dev)
    y, loss, dW, dX = tnn.train_step_l2(desc, pf, pb, xt, tt, ls)
    # the same step from the separate entry points
    interm_t = tnn.forward(desc, pf, xt)
    values, grads = tnn.l2_loss(dtype, interm_t[-1], tt, ls)
    _, dW_u, dX_u = tnn.backward(desc, pb, grads, interm_t, dw_fp32=True)
    assert torch.equal(y, interm_t[-1])  # same kernel arithmetic: bit-identical outputs
    assert torch.equal(dX, dX_u)
    assert abs(float(loss.item()) - float(values.sum().item())) <= 1e-5 * float(values.sum().item())
    dWh, dWu = tnn.host(dW), tnn.host(dW_u)
    assert np.abs(dWh - dWu).max() <= 1e-5 * np.abs(dWu).max() + 1e-9  # fp32 sums in a different order
    # and against the oracle (backward fed the GPU's activations)
    interm = tnn.host(interm_t)
    rv, rg = oracle.l2_loss(dtype, interm[-1], targets, ls)
    assert np.array_equal(tnn.host(grads), rg)
    _, rdW, rdX = oracle.mlp_backward_T(dtype, W, n_mats, act, out_act, w, interm, rg, round_dw=False)
    assert_propagated(dWh, rdW, dtype, "dW", scale=float(np.abs(rdW).max()))
    assert_propagated(tnn.host(dX), rdX, dtype, "dL/dx", scale=float(np.abs(rdX).max()))
    # optional outputs can be left out
    y2, loss2, dW2, dX2 = tnn.train_step_l2(desc, pf, pb, xt, tt, ls, want_y=False, want_dx=False, dw_fp32=False)
    assert y2 is None and dX2 is None
    assert np.array_equal(tnn.host(dW2), oracle.round(dWh, dtype))


@pytest.mark.parametrize("W,n_hidden", [(16, 2), (32, 4), (128, 8)])
def test_baseline_config_3_full_size(tnn, oracle, W, n_hidden):
    """BASELINE config 3: fp16, batch 2^20, as inference and as a training step. Inference: a seeded sample of 4096 rows
    against the oracle, and the rows of a sub-batch bit-identical to the same rows inside the full batch. Training step:
    the loss-scaled weight gradients of the whole batch equal the sum over its two halves (the gradient is additive over
    rows; fp32 sums in another order), the halves' network outputs are the full batch's rows, and a sampled sub-batch's
    gradients match the oracle."""
    import torch
    dtype, M = FP16, 1 << 20
    n_mats = n_hidden + 1
    w = oracle.round(xavier(W, n_mats, 3), dtype)
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    _, pf, pb = tnn.prepare(desc, w)
    gen = torch.Generator(device=tnn.dev).manual_seed(33)
    x = (torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1).to(torch.float16)
    y = tnn.inference(desc, pf, x)
    sel = torch.sort(torch.randperm(M, device=tnn.dev, generator=gen)[:4096]).values
    ref = oracle.mlp_forward_T(dtype, W, n_mats, "relu", "none", w, x[sel].float().cpu().numpy(), store_interm=False)
    assert_propagated(y[sel].float().cpu().numpy(), ref, dtype, "config 3 inference, sampled rows")
    assert torch.equal(tnn.inference(desc, pf, x[4096:3 * 4096].contiguous()), y[4096:3 * 4096])

    targets = torch.rand((M, W), device=tnn.dev, generator=gen)
    loss_scale = 128.0 * (M / 1024)  # keeps dL/dy = loss_scale * 2 (y - t) / (M W) clear of fp16's denormal range
    yf, lf, dWf, _ = tnn.train_step_l2(desc, pf, pb, x, targets, loss_scale, want_dx=False)
    assert torch.equal(yf, y)
    h = M // 2
    # a half batch averages over half as many elements: half the loss scale gives the same per-row gradient
    ya, la, dWa, _ = tnn.train_step_l2(desc, pf, pb, x[:h].contiguous(), targets[:h].contiguous(), loss_scale / 2, want_dx=False)
    yb, lb, dWb, _ = tnn.train_step_l2(desc, pf, pb, x[h:].contiguous(), targets[h:].contiguous(), loss_scale / 2, want_dx=False)
    assert torch.equal(ya, y[:h]) and torch.equal(yb, y[h:])
    full, parts = dWf.double().cpu().numpy(), (dWa.double() + dWb.double()).cpu().numpy()
    assert np.abs(full - parts).max() <= 1e-4 * np.abs(full).max()
    assert abs(float(lf) - 0.5 * (float(la) + float(lb))) <= 1e-5 * float(lf)
    # a sub-batch small enough for the oracle
    S = 2048
    xs, ts = x[:S].contiguous(), targets[:S].contiguous()
    ys_, ls, dWs, dXs = tnn.train_step_l2(desc, pf, pb, xs, ts, 4096.0)
    interm = oracle.mlp_forward_T(dtype, W, n_mats, "relu", "none", w, xs.float().cpu().numpy())
    _, grads = oracle.l2_loss(dtype, interm[-1], ts.cpu().numpy(), 4096.0)
    _, rdW, rdX = oracle.mlp_backward_T(dtype, W, n_mats, "relu", "none", w, interm, grads, round_dw=False)
    assert_propagated(dWs.cpu().numpy(), rdW, dtype, "dW of the sub-batch", scale=float(np.abs(rdW).max()))
    # dL/dx has up to nine rounded ReLU layers behind it, forward and backward (the step does not expose its activations,
    # so the oracle runs on its own), and no sum over the batch to average a flipped mask out: a row in which one
    # pre-activation rounds to the other side of zero gets the other mask and differs in all of its elements (0.5 % of
    # the rows at width 128 with 8 hidden layers). 98 % of the rows must be inside the elementwise bar in every element,
    # and the whole matrix within 2e-2 in the Frobenius norm (1.2e-2 measured).
    dXh = dXs.float().cpu().numpy()
    diff, bar = np.abs(dXh - rdX), 5e-4 * np.abs(rdX).max() + 5e-3 * np.abs(rdX)
    assert (diff <= bar).all(axis=1).mean() >= 0.98
    assert np.linalg.norm((dXh - rdX).ravel()) <= 2e-2 * np.linalg.norm(rdX.ravel())
    # The same gradients at the bar of every other end-to-end check, with the masks taken out of the comparison: the oracle's
    # backward pass over the activations the GPU's forward pass stores (the step's own, bit for bit: same kernel, and its
    # output is checked to be theirs), so both sides gate with the same ReLU masks and differ only by the rounding of the deltas.
    interm_t = tnn.forward(desc, pf, xs)
    assert torch.equal(ys_, interm_t[-1])
    interm_g = tnn.host(interm_t)
    _, grads_g = oracle.l2_loss(dtype, interm_g[-1], ts.cpu().numpy(), 4096.0)
    _, rdW_g, rdX_g = oracle.mlp_backward_T(dtype, W, n_mats, "relu", "none", w, interm_g, grads_g, round_dw=False)
    assert_propagated(dXh, rdX_g, dtype, "dL/dx of the sub-batch over the GPU's activations", scale=float(np.abs(rdX_g).max()))
    assert_propagated(dWs.cpu().numpy(), rdW_g, dtype, "dW of the sub-batch over the GPU's activations", scale=float(np.abs(rdW_g).max()))


@pytest.mark.parametrize("dtype,n_hidden,act,out_act,M", [(FP16, 8, "relu", "none", (1 << 16) + 8 * 37), (BF16, 3, "relu", "sigmoid", 1 << 16),
                                                          (FP16, 2, "sigmoid", "none", (1 << 17) + 8), (BF16, 5, "relu", "relu", (1 << 16) + 2048)])
def test_width_128_step_without_stored_output(tnn, oracle, dtype, n_hidden, act, out_act, M):
    """A width-128 training step that is not asked for the network's output ends its forward pass at the last hidden layer;
    the top launch of its backward pass forms the output again with the forward pass's arithmetic. Everything it returns
    must be what the step with the output stored returns: dL/dx bit for bit, the weight gradients bit for bit as well (same
    partial sums over the same values), the loss to the rounding of its sum. Odd and even numbers of matrices (the bottom
    layer alone or in a pair), ragged last rounds, every output activation; the batch sizes are those of the streaming
    forward kernel (the small ones are in test_train_step_single_call)."""
    import torch
    W, n_mats = 128, n_hidden + 1
    w = oracle.round(xavier(W, n_mats, 11), dtype)
    desc = tnn.mlp_desc(dtype, W, n_hidden, act, out_act)
    _, pf, pb = tnn.prepare(desc, w)
    gen = torch.Generator(device=tnn.dev).manual_seed(21)
    x = (torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1).to(torch.float16 if dtype == FP16 else torch.bfloat16)
    targets = torch.rand((M, W), device=tnn.dev, generator=gen)
    ls = 128.0 * M / 1024
    y, loss, dW, dX = tnn.train_step_l2(desc, pf, pb, x, targets, ls, want_y=True, want_dx=True, dw_fp32=True)
    y2, loss2, dW2, dX2 = tnn.train_step_l2(desc, pf, pb, x, targets, ls, want_y=False, want_dx=True, dw_fp32=True)
    assert y2 is None
    assert torch.equal(dX2.view(torch.int16), dX.view(torch.int16))
    assert torch.equal(dW2.view(torch.int32), dW.view(torch.int32))
    assert abs(float(loss2) - float(loss)) <= 1e-6 * abs(float(loss))
    # the step with the optimizer inside takes the same route: one step from zero moments against the oracle's Adam on dW
    from gpu_harness import ptr
    from tiny_dpcpp_nn import _lib
    master = tnn.pack(FP32, W, n_mats, torch.from_numpy(w.reshape(-1)).to(tnn.dev))
    dWp = torch.empty(n_mats * W * W, dtype=torch.float32, device=tnn.dev)
    _lib.check(tnn.lib.tnn_pack_and_transpose(2, W, n_mats, ptr(dW), ptr(dWp), tnn.stream()))
    rp, rm, rv = oracle.adam_step(tnn.host(master), np.zeros(master.numel(), np.float32), np.zeros(master.numel(), np.float32),
                                  tnn.host(dWp) / np.float32(ls), 1, 1e-2, 0.9, 0.999, 1e-8)
    pf2, pb2 = tnn.prepare_packed(desc, master, src_is_fp32=True)
    m, v = torch.zeros_like(master), torch.zeros_like(master)
    ws_bytes = tnn.lib.tnn_mlp_train_step_workspace_bytes(ctypes.byref(desc), M)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=tnn.dev)
    loss3 = torch.full((1,), float("nan"), device=tnn.dev)
    _lib.check(tnn.lib.tnn_mlp_train_step_l2_adam(ctypes.byref(desc), ptr(pf2), ptr(pb2), ptr(x), ptr(targets), ls, None, ptr(loss3), ptr(master),
                                                  ptr(m), ptr(v), 1, 1e-2, 0.9, 0.999, 1e-8, None, None, M, ptr(ws), ws_bytes, None, tnn.stream()))
    tnn.sync()
    assert abs(float(loss3) - float(loss)) <= 1e-6 * abs(float(loss))
    assert np.allclose(tnn.host(m), rm, rtol=1e-5, atol=1e-12) and np.allclose(tnn.host(v), rv, rtol=1e-5, atol=1e-20)
    assert np.allclose(tnn.host(master), rp, rtol=1e-6, atol=2e-6)
    wf_ref, wb_ref = tnn.prepare_packed(desc, master, src_is_fp32=True)
    assert torch.equal(pf2.view(torch.int16), wf_ref.view(torch.int16)) and torch.equal(pb2.view(torch.int16), wb_ref.view(torch.int16))


@pytest.mark.parametrize("dtype,W,n_hidden,log2_m", [(FP16, 16, 2, 19), (FP16, 16, 4, 19), (BF16, 32, 2, 19), (BF16, 64, 4, 18), (FP16, 64, 2, 17)])
def test_train_step_is_reproducible(tnn, oracle, dtype, W, n_hidden, log2_m):
    """The same step on the same data gives the same bits, every time: the partial sums are added in a fixed order and
    nothing in the kernel depends on timing. Batches of several rounds per wave; width 16 is the shape in which half of
    every weight-gradient accumulator is unused, which is where a register written behind the compiler's back (inline asm
    next to an MFMA in flight) once made the result vary from run to run."""
    import torch
    M, n_mats = 1 << log2_m, n_hidden + 1
    w = oracle.round(xavier(W, n_mats, 5), dtype)
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    _, pf, pb = tnn.prepare(desc, w)
    gen = torch.Generator(device=tnn.dev).manual_seed(9)
    x = (torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1).to(torch.float16 if dtype == FP16 else torch.bfloat16)
    targets = torch.rand((M, W), device=tnn.dev, generator=gen)
    first = None
    for _ in range(4):
        y, loss, dW, dX = tnn.train_step_l2(desc, pf, pb, x, targets, 128.0 * M / 1024, want_dx=True, dw_fp32=True)
        tnn.sync()
        got = (y.clone(), loss.clone(), dW.clone(), dX.clone())
        if first is None:
            first = got
        else:
            for a, b in zip(got, first):
                assert torch.equal(a.view(torch.int16 if a.element_size() == 2 else torch.int32), b.view(torch.int16 if b.element_size() == 2 else torch.int32))


@pytest.mark.parametrize("dtype,W,n_hidden,act,out_act,M", [
    (BF16, 64, 4, "relu", "none", 1 << 14), (BF16, 64, 4, "relu", "none", 8), (FP16, 64, 2, "relu", "relu", 4104),
    (FP16, 64, 1, "sigmoid", "sigmoid", 1000 * 8), (BF16, 32, 4, "relu", "none", 3 * 4096 + 8), (FP16, 32, 5, "none", "none", 2048),
    (FP16, 16, 2, "relu", "sigmoid", 777 * 8), (BF16, 16, 5, "sigmoid", "none", 4096)])
def test_backward_recompute_equals_forward_plus_backward(tnn, oracle, dtype, W, n_hidden, act, out_act, M):
    """The backward pass that forms the activations again on chip (tnn_mlp_backward_recompute, the backward half of a training
    step whose loss the caller computes) against forward_pass + backward_pass on the same inputs: dL/dx bit for bit (the same
    rounded chain per row), the weight gradients to the rounding of fp32 sums taken in another order, and both against the
    oracle (Network::backward_pass, include/network/kernel_esimd.h:160-240)."""
    import torch
    n_mats = n_hidden + 1
    w, x = make_case(oracle, dtype, W, n_mats, M)
    rng = np.random.default_rng(M + W)
    g = oracle.round(rng.standard_normal((M, W)) * 0.05, dtype)
    desc = tnn.mlp_desc(dtype, W, n_hidden, act, out_act)
    assert tnn.lib.tnn_mlp_backward_recompute_supported(ctypes.byref(desc)) == 0
    _, pf, pb = tnn.prepare(desc, w)
    xt, gt = tnn.dev_tensor(x, dtype), tnn.dev_tensor(g, dtype)
    interm = tnn.forward(desc, pf, xt)
    _, dW_ref, dX_ref = tnn.backward(desc, pb, gt, interm, dw_fp32=True)
    dW, dX = tnn.backward_recompute(desc, pf, pb, xt, gt)
    assert torch.equal(dX.view(torch.int16), dX_ref.view(torch.int16)), "dL/dx differs from forward_pass + backward_pass"
    scale = float(dW_ref.abs().max())
    assert torch.allclose(dW, dW_ref, rtol=1e-4, atol=1e-5 * scale), float((dW - dW_ref).abs().max())
    ri = oracle.mlp_forward_T(dtype, W, n_mats, act, out_act, w, x)
    _, rdW, rdX = oracle.mlp_backward_T(dtype, W, n_mats, act, out_act, w, ri, g, round_dw=False)
    assert_propagated(tnn.host(dW), rdW, dtype, "dW of the recompute backward", scale=float(np.abs(rdW).max()))
    assert_close(tnn.host(dX), rdX, dtype, "dL/dx of the recompute backward", scale=float(np.abs(rdX).max()), frac_ok=PROPAGATED)
    # without dL/dx, and with the gradients in the network's type
    dW2, none = tnn.backward_recompute(desc, pf, pb, xt, gt, want_dx=False, dw_fp32=False)
    assert none is None and torch.equal(dW2.view(torch.int16), dW.to(dW2.dtype).view(torch.int16))


def test_backward_recompute_rejects_what_it_cannot_run(tnn):
    from tiny_dpcpp_nn import _lib
    wide = tnn.mlp_desc(FP16, 128, 2, "relu", "none")
    deep = tnn.mlp_desc(BF16, 64, 7, "relu", "none")
    for d in (wide, deep):
        assert tnn.lib.tnn_mlp_backward_recompute_supported(ctypes.byref(d)) == _lib.TNN_ERR_UNSUPPORTED
    ok = tnn.mlp_desc(BF16, 64, 2, "relu", "none")
    import torch
    t = torch.zeros((8, 64), dtype=torch.bfloat16, device=tnn.dev)
    ws = torch.empty(16, dtype=torch.uint8, device=tnn.dev)
    from gpu_harness import ptr
    assert tnn.lib.tnn_mlp_backward_recompute(ctypes.byref(ok), ptr(t), ptr(t), ptr(t), ptr(t), ptr(t), 1, None, 8, ptr(ws), 16, tnn.stream()) == _lib.TNN_ERR_WORKSPACE
    assert tnn.lib.tnn_mlp_backward_recompute(ctypes.byref(ok), ptr(t), ptr(t), ptr(t), None, ptr(t), 1, None, 8, ptr(ws), 16, tnn.stream()) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert tnn.lib.tnn_mlp_backward_recompute(ctypes.byref(ok), ptr(t), ptr(t), ptr(t), ptr(t), ptr(t), 1, None, 12, ptr(ws), 16, tnn.stream()) == _lib.TNN_ERR_INVALID_ARGUMENT
