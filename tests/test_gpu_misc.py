"""L2 loss and Adam kernels against the oracle."""
import numpy as np
import pytest
import torch

from tolerances import BF16, FP16, FP32

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,tdt", [(BF16, torch.bfloat16), (FP16, torch.float16)])
def test_l2_loss(tnn, oracle, dtype, tdt):
    rng = np.random.default_rng(0)
    M, W = 1024, 64
    pred = oracle.round(rng.standard_normal((M, W)), dtype)
    targ = rng.uniform(0, 1, (M, W)).astype(np.float32)
    for ls in (1.0, 128.0, 10.0):
        values, grads = tnn.l2_loss(dtype, torch.from_numpy(pred).to(tnn.dev).to(tdt), torch.from_numpy(targ).to(tnn.dev), ls)
        rv, rg = oracle.l2_loss(dtype, pred, targ, ls)
        assert np.allclose(values.cpu().numpy(), rv, rtol=1e-6, atol=0)
        assert np.array_equal(tnn.host(grads), rg)  # same fp32 expression, same rounding: bit-exact
    # closed form of test/doctest_losses.cpp:46-51
    p = torch.full((8, 16), 0.5, device=tnn.dev).to(tdt)
    t = torch.full((8, 16), 0.125, device=tnn.dev)
    values, grads = tnn.l2_loss(dtype, p, t, 4.0)
    assert np.allclose(values.cpu().numpy(), 0.375 ** 2 / 128)
    assert np.allclose(tnn.host(grads), 4.0 * 2 * 0.375 / 128, rtol=4e-3)


@pytest.mark.parametrize("dtype", [BF16, FP16, FP32])
def test_fill_uniform(tnn, oracle, dtype):
    """The seeded initialiser (default grid table, Xavier weights) equals the oracle's restatement bit for bit, whatever the
    size of the launch, and an offset into the sequence continues it."""
    from tiny_dpcpp_nn import _lib
    from tiny_dpcpp_nn.cabi import ptr
    for n, lo, hi, seed, first in ((1, -1.0, 1.0, 0, 0), (100003, -1e-4, 1e-4, 777, 0), (1 << 22, -0.2165, 0.2165, 2 ** 63 + 5, 2 ** 40)):
        t = tnn.empty((n,), dtype, fill=float("nan"))
        _lib.check(tnn.lib.tnn_fill_uniform(dtype, ptr(t), n, lo, hi, seed, first, tnn.stream()))
        assert np.array_equal(tnn.host(t), oracle.fill_uniform(n, lo, hi, seed, first, dtype))
    a, b = tnn.empty((1000,), FP32), tnn.empty((400,), FP32)
    _lib.check(tnn.lib.tnn_fill_uniform(FP32, ptr(a), 1000, 0.0, 1.0, 3, 0, tnn.stream()))
    _lib.check(tnn.lib.tnn_fill_uniform(FP32, ptr(b), 400, 0.0, 1.0, 3, 600, tnn.stream()))
    assert torch.equal(a[600:], b)
    assert tnn.lib.tnn_fill_uniform(FP32, ptr(a), 10, 1.0, 0.0, 3, 0, tnn.stream()) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert tnn.lib.tnn_fill_uniform(7, ptr(a), 10, 0.0, 1.0, 3, 0, tnn.stream()) == _lib.TNN_ERR_UNSUPPORTED


def test_adam(tnn, oracle):
    rng = np.random.default_rng(1)
    n = 20480
    p0 = rng.standard_normal(n).astype(np.float32) * 0.1
    p = torch.from_numpy(p0.copy()).to(tnn.dev)
    m = torch.zeros_like(p)
    v = torch.zeros_like(p)
    rp, rm, rv = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    tp = torch.nn.Parameter(torch.from_numpy(p0.copy()))
    opt = torch.optim.Adam([tp], lr=1e-3, betas=(0.9, 0.99), eps=1e-15)
    pT = torch.empty(n, dtype=torch.float16, device=tnn.dev)
    for step in range(1, 5):
        g = (rng.standard_normal(n) * 128).astype(np.float32)
        gs = 1.0 / 128
        tnn.adam_step(p, m, v, torch.from_numpy(g).to(tnn.dev), FP32, gs, step, 1e-3, 0.9, 0.99, 1e-15, pT, FP16)
        rp, rm, rv = oracle.adam_step(rp, rm, rv, g * np.float32(gs), step, 1e-3, 0.9, 0.99, 1e-15)
        tp.grad = torch.from_numpy(g * np.float32(gs))
        opt.step()
        assert np.allclose(tnn.host(p), rp, rtol=1e-6, atol=1e-7)
        assert np.allclose(tnn.host(p), tp.detach().numpy(), rtol=1e-6, atol=1e-7)
    assert np.array_equal(tnn.host(pT), oracle.round(tnn.host(p), FP16))
    # half-precision gradients
    g16 = oracle.round(rng.standard_normal(n), BF16)
    tnn.adam_step(p, m, v, torch.from_numpy(g16).to(tnn.dev).to(torch.bfloat16), BF16, 1.0, 5, 1e-3, 0.9, 0.99, 1e-15)
    rp, rm, rv = oracle.adam_step(rp, rm, rv, g16, 5, 1e-3, 0.9, 0.99, 1e-15)
    assert np.allclose(tnn.host(p), rp, rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("dtype,tdt", [(BF16, torch.bfloat16), (FP16, torch.float16)])
@pytest.mark.parametrize("W,n_hidden", [(64, 4), (16, 2), (32, 3), (128, 1)])
def test_fused_adam_update_equals_the_three_separate_calls(tnn, dtype, tdt, W, n_hidden):
    """tnn_mlp_adam_update == tnn_pack_and_transpose + tnn_adam_step + tnn_mlp_prepare_weights, bit for bit."""
    import ctypes
    from gpu_harness import ptr
    from tiny_dpcpp_nn import _lib
    n_mats = n_hidden + 1
    n = n_mats * W * W
    gen = torch.Generator(device=tnn.dev).manual_seed(W + n_hidden)
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    master = torch.randn(n, device=tnn.dev, generator=gen) * 0.1
    m0 = torch.randn(n, device=tnn.dev, generator=gen) * 0.01
    v0 = torch.rand(n, device=tnn.dev, generator=gen) * 0.01
    dW = torch.randn((n_mats, W, W), device=tnn.dev, generator=gen)
    # separate calls
    p1, m1, v1 = master.clone(), m0.clone(), v0.clone()
    gp = torch.empty(n, device=tnn.dev)
    _lib.check(tnn.lib.tnn_pack_and_transpose(FP32, W, n_mats, ptr(dW), ptr(gp), tnn.stream()))
    pT1 = torch.empty(n, dtype=tdt, device=tnn.dev)
    tnn.adam_step(p1, m1, v1, gp, FP32, 1.0 / 128, 3, 1e-3, 0.9, 0.99, 1e-15, pT1, dtype)
    f1, b1 = tnn.prepare_packed(desc, p1, src_is_fp32=True)
    # one call; the operand buffers start from a prepared state (their zero padding is never rewritten)
    p2, m2, v2 = master.clone(), m0.clone(), v0.clone()
    f2, b2 = tnn.prepare_packed(desc, master, src_is_fp32=True)
    pT2 = torch.empty(n, dtype=tdt, device=tnn.dev)
    _lib.check(tnn.lib.tnn_mlp_adam_update(ctypes.byref(desc), ptr(p2), ptr(m2), ptr(v2), ptr(dW), 1.0 / 128, 3, 1e-3, 0.9, 0.99, 1e-15,
                                           ptr(pT2), ptr(f2), ptr(b2), tnn.stream()))
    for a, b in ((p1, p2), (m1, m2), (v1, v2), (pT1, pT2), (f1, f2), (b1, b2)):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype,tdt", [(BF16, torch.bfloat16), (FP16, torch.float16)])
@pytest.mark.parametrize("W,n_hidden,M", [(64, 4, 8192), (16, 2, 1000 * 8), (32, 5, 4096), (128, 2, 2048), (64, 6, 2048)])
def test_train_step_with_adam_equals_step_then_update(tnn, dtype, tdt, W, n_hidden, M):
    """tnn_mlp_train_step_l2_adam == tnn_mlp_train_step_l2 (fp32 gradients) + tnn_mlp_adam_update, bit for bit: the same
    reduction order produces the same gradient sums, the same per-weight arithmetic follows. Covers shapes with the fused
    kernel and shapes without one (width 128, or too deep), and two steps in a row (the second reads the re-staged weights)."""
    import ctypes
    from gpu_harness import ptr
    from tiny_dpcpp_nn import _lib
    n_mats = n_hidden + 1
    n = n_mats * W * W
    gen = torch.Generator(device=tnn.dev).manual_seed(W * 7 + n_hidden)
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    d = ctypes.byref(desc)
    master = (torch.rand(n, device=tnn.dev, generator=gen) * 2 - 1) * (6.0 / (2 * W)) ** 0.5
    x = (torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1).to(tdt)
    targets = torch.rand((M, W), device=tnn.dev, generator=gen)
    loss_scale = 128.0 if dtype == FP16 else 1.0
    ws_bytes = tnn.lib.tnn_mlp_train_step_workspace_bytes(d, M)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=tnn.dev)
    hyper = (1e-2, 0.9, 0.99, 1e-15)

    def fresh():
        f, b = tnn.prepare_packed(desc, master, src_is_fp32=True)
        return dict(p=master.clone(), m=torch.zeros(n, device=tnn.dev), v=torch.zeros(n, device=tnn.dev), f=f, b=b,
                    pT=torch.empty(n, dtype=tdt, device=tnn.dev), y=torch.empty_like(x), dx=torch.empty_like(x),
                    loss=torch.zeros(1, device=tnn.dev))

    a, b = fresh(), fresh()
    dW = torch.empty((n_mats, W, W), device=tnn.dev)
    for step in (1, 2):
        _lib.check(tnn.lib.tnn_mlp_train_step_l2(d, ptr(a["f"]), ptr(a["b"]), ptr(x), ptr(targets), loss_scale, ptr(a["y"]), ptr(a["loss"]),
                                                 ptr(dW), 1, ptr(a["dx"]), M, ptr(ws), ws_bytes, tnn.stream()))
        _lib.check(tnn.lib.tnn_mlp_adam_update(d, ptr(a["p"]), ptr(a["m"]), ptr(a["v"]), ptr(dW), 1.0 / loss_scale, step, *hyper,
                                               ptr(a["pT"]), ptr(a["f"]), ptr(a["b"]), tnn.stream()))
        _lib.check(tnn.lib.tnn_mlp_train_step_l2_adam(d, ptr(b["f"]), ptr(b["b"]), ptr(x), ptr(targets), loss_scale, ptr(b["y"]),
                                                      ptr(b["loss"]), ptr(b["p"]), ptr(b["m"]), ptr(b["v"]), step, *hyper, ptr(b["pT"]),
                                                      ptr(b["dx"]), M, ptr(ws), ws_bytes, None, tnn.stream()))
        torch.cuda.synchronize()
        for key in ("y", "dx", "p", "m", "v", "pT", "f", "b"):
            assert torch.equal(a[key], b[key]), f"step {step}: {key} differs"
        # shapes without the fused kernel add the loss up with float atomics, in an order that changes from run to run
        assert torch.allclose(a["loss"], b["loss"], rtol=1e-5, atol=0), f"step {step}: loss differs"
    assert not torch.equal(a["p"], master)   # the weights did move
    # argument checks
    assert tnn.lib.tnn_mlp_train_step_l2_adam(d, ptr(b["f"]), ptr(b["b"]), ptr(x), ptr(targets), loss_scale, None, None, ptr(b["p"]),
                                              ptr(b["m"]), ptr(b["v"]), 0, *hyper, None, None, M, ptr(ws), ws_bytes, None,
                                              tnn.stream()) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert tnn.lib.tnn_mlp_train_step_l2_adam(d, ptr(b["f"]), ptr(b["b"]), ptr(x), ptr(targets), loss_scale, None, None, ptr(b["p"]),
                                              ptr(b["m"]), ptr(b["v"]), 1, *hyper, None, None, M, ptr(ws), 16, None,
                                              tnn.stream()) == _lib.TNN_ERR_WORKSPACE


def test_two_streams_give_the_single_stream_results(tnn):
    """The library keeps no state between calls: calls enqueued on two streams (a network each, its own buffers) give bit
    for bit what the same calls give one after the other on one stream. Both streams have the default priority."""
    import ctypes

    from gpu_harness import ptr
    from tiny_dpcpp_nn import _lib

    gen = torch.Generator(device=tnn.dev).manual_seed(3)
    cases = []
    for dtype, tdt, W, n_hidden, M in ((BF16, torch.bfloat16, 64, 4, 1 << 16), (FP16, torch.float16, 32, 2, (1 << 16) + 8)):
        n_mats = n_hidden + 1
        desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
        master = (torch.rand(n_mats * W * W, device=tnn.dev, generator=gen) * 2 - 1) * (6.0 / (2 * W)) ** 0.5
        pf, pb = tnn.prepare_packed(desc, master, src_is_fp32=True)
        x = (torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1).to(tdt)
        g = ((torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1) / M).to(tdt)
        ws_bytes = tnn.lib.tnn_mlp_backward_workspace_bytes(ctypes.byref(desc), M)
        cases.append(dict(desc=desc, pf=pf, pb=pb, x=x, g=g, M=M, W=W, n_mats=n_mats, tdt=tdt, ws_bytes=ws_bytes))

    def run(case, stream):
        c, d = case, ctypes.byref(case["desc"])
        s = ctypes.c_void_p(stream.cuda_stream)
        out = dict(y=torch.empty_like(c["x"]), interm=torch.empty((c["n_mats"] + 1, c["M"], c["W"]), dtype=c["tdt"], device=tnn.dev),
                   ib=torch.empty((c["n_mats"], c["M"], c["W"]), dtype=c["tdt"], device=tnn.dev),
                   dW=torch.empty(c["n_mats"] * c["W"] * c["W"], dtype=torch.float32, device=tnn.dev), dX=torch.empty_like(c["x"]),
                   ws=torch.empty(c["ws_bytes"], dtype=torch.uint8, device=tnn.dev))
        for _ in range(3):  # several rounds so that the two streams really overlap
            _lib.check(tnn.lib.tnn_mlp_inference(d, ptr(c["pf"]), ptr(c["x"]), ptr(out["y"]), c["M"], s))
            _lib.check(tnn.lib.tnn_mlp_forward(d, ptr(c["pf"]), ptr(c["x"]), ptr(out["interm"]), c["M"], s))
            _lib.check(tnn.lib.tnn_mlp_backward(d, ptr(c["pb"]), ptr(c["g"]), ptr(out["interm"]), ptr(out["ib"]), ptr(out["dW"]), 1,
                                                ptr(out["dX"]), c["M"], ptr(out["ws"]), c["ws_bytes"], s))
        return out

    torch.cuda.synchronize()
    one = torch.cuda.current_stream()
    ref = [run(c, one) for c in cases]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [run(c, st) for c, st in zip(cases, streams)]
    torch.cuda.synchronize()
    for r, o in zip(ref, got):
        for k in ("y", "interm", "ib", "dW", "dX"):
            assert torch.equal(r[k], o[k]), k


def test_two_host_threads(tnn):
    """Two host threads, a stream each, call the library at the same time (ctypes releases the GIL during a call): same
    results as one thread. What the library caches per device lives in thread-local storage."""
    import ctypes
    import threading

    from gpu_harness import ptr
    from tiny_dpcpp_nn import _lib

    gen = torch.Generator(device=tnn.dev).manual_seed(4)
    W, n_hidden, M = 64, 3, 1 << 15
    desc = tnn.mlp_desc(BF16, W, n_hidden, "relu", "none")
    master = (torch.rand((n_hidden + 1) * W * W, device=tnn.dev, generator=gen) * 2 - 1) * 0.2
    pf, _ = tnn.prepare_packed(desc, master, src_is_fp32=True)
    xs = [(torch.rand((M, W), device=tnn.dev, generator=gen) * 2 - 1).to(torch.bfloat16) for _ in range(2)]
    ref = [tnn.inference(desc, pf, x) for x in xs]
    torch.cuda.synchronize()
    outs = [torch.empty_like(x) for x in xs]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    errors = []

    def worker(i):
        try:
            s = ctypes.c_void_p(streams[i].cuda_stream)
            for _ in range(200):
                _lib.check(tnn.lib.tnn_mlp_inference(ctypes.byref(desc), ptr(pf), ptr(xs[i]), ptr(outs[i]), M, s))
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for r, o in zip(ref, outs):
        assert torch.equal(r, o)


def test_a_meeting_that_gives_up_poisons_the_step(tnn, oracle):
    """The waves of the width-64 training kernels meet at an LDS counter with a bounded wait. With the bound forced to 0
    from the host every wait gives up at once; every kernel still runs to its end, and the call must then return NaN in
    the loss and in every weight gradient, never a plausible number. Back at the default bound the same call is right."""
    import torch
    from gpu_harness import ptr
    from tiny_dpcpp_nn import _lib
    dtype, W, n_hidden, M = BF16, 64, 4, 1 << 17  # two rounds per wave: the first has meetings
    n_mats = n_hidden + 1
    rng = np.random.default_rng(5)
    lim = np.sqrt(6.0 / (2 * W))
    w = oracle.round(rng.uniform(-lim, lim, (n_mats, W, W)), dtype)
    x = oracle.round(rng.uniform(-1, 1, (M, W)), dtype)
    desc = tnn.mlp_desc(dtype, W, n_hidden, "relu", "none")
    _, pf, pb = tnn.prepare(desc, w)
    xt = tnn.dev_tensor(x, dtype)
    tt = torch.from_numpy(rng.uniform(0, 1, (M, W)).astype(np.float32)).to(tnn.dev)
    good = tnn.train_step_l2(desc, pf, pb, xt, tt, 1.0)
    torch.cuda.synchronize()
    import ctypes
    before = ctypes.c_int(-1)
    assert tnn.lib.tnn_debug_set_meeting_spin_limit(0, ctypes.byref(before)) == _lib.TNN_OK
    old = before.value
    try:
        assert old == 1 << 22
        y, loss, dW, dX = tnn.train_step_l2(desc, pf, pb, xt, tt, 1.0)
        interm = tnn.forward(desc, pf, xt)
        g = (torch.rand((M, W), device=tnn.dev) / M).to(torch.bfloat16)
        _, dW_b, dX_b = tnn.backward(desc, pb, g, interm, dw_fp32=True)
        torch.cuda.synchronize()
    finally:
        assert tnn.lib.tnn_debug_set_meeting_spin_limit(old, ctypes.byref(before)) == _lib.TNN_OK and before.value == 0
    assert torch.isnan(loss).all() and torch.isnan(dW).all(), "a step whose waits gave up must not return numbers"
    assert torch.isnan(dW_b).all()
    # what does not depend on other waves' tiles is still right
    assert torch.equal(y.view(torch.int16), good[0].view(torch.int16)) and torch.equal(dX.view(torch.int16), good[3].view(torch.int16))
    again = tnn.train_step_l2(desc, pf, pb, xt, tt, 1.0)
    torch.cuda.synchronize()
    for a, b in zip(again, good):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    assert tnn.lib.tnn_debug_set_meeting_spin_limit(-1, None) == _lib.TNN_ERR_INVALID_ARGUMENT
    assert tnn.lib.tnn_debug_set_meeting_spin_limit(1 << 22, ctypes.byref(before)) == _lib.TNN_OK and before.value == 1 << 22
