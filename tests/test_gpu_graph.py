"""The entry points only enqueue kernels (no memset nodes, no allocation, no synchronisation), so a caller can record them
into a HIP graph. A step of BASELINE config 4's shape (encoding forward, fused training step, scatter into the gradient
table with Overwrite) is captured once and replayed on changing inputs; every replay is compared with the eager result,
with the program's own eager work between the replays. The reference offers the same for its training step through
SyclGraph (include/trainer.h:27-31, source/common/SyclGraph.cpp:44-86)."""
import ctypes

import pytest
import torch

from gpu_harness import ptr
from tiny_dpcpp_nn import _lib
from tolerances import FP16, FP32

pytestmark = pytest.mark.gpu

CFG = dict(n_dims=2, n_levels=16, n_features_per_level=2, log2_hashmap_size=15, base_resolution=16, per_level_scale=1.5)
W = 64


def test_captured_step_replays_like_eager(tnn):
    M, n_hidden = 1 << 14, 2
    n_mats = n_hidden + 1
    gen = torch.Generator(device=tnn.dev).manual_seed(9)
    gd = tnn.grid_desc(CFG, FP16)
    n_table = tnn.grid_n_params(gd)
    table = (torch.rand(n_table, device=tnn.dev, generator=gen) * 2 - 1).to(torch.float16)
    desc = tnn.mlp_desc(FP16, W, n_hidden, "relu", "none")
    d = ctypes.byref(desc)
    master = (torch.rand(n_mats * W * W, device=tnn.dev, generator=gen) * 2 - 1) * 0.2
    pf, pb = tnn.prepare_packed(desc, master, src_is_fp32=True)
    x = torch.rand((M, 2), device=tnn.dev, generator=gen)
    targets = torch.rand((M, W), device=tnn.dev, generator=gen)
    enc = torch.empty((M, W), dtype=torch.float16, device=tnn.dev)
    denc = torch.empty_like(enc)
    y = torch.empty_like(enc)
    dW = torch.empty((n_mats, W, W), device=tnn.dev)
    loss = torch.zeros(1, device=tnn.dev)
    grad_table = torch.empty(n_table, device=tnn.dev)
    ws_bytes = tnn.lib.tnn_mlp_train_step_workspace_bytes(d, M)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=tnn.dev)

    def step():
        s = tnn.stream()
        _lib.check(tnn.lib.tnn_grid_forward(ctypes.byref(gd), ptr(x), ptr(table), ptr(enc), FP16, W, M, s))
        _lib.check(tnn.lib.tnn_mlp_train_step_l2(d, ptr(pf), ptr(pb), ptr(enc), ptr(targets), 4096.0, ptr(y), ptr(loss), ptr(dW), 1,
                                                 ptr(denc), M, ptr(ws), ws_bytes, s))
        _lib.check(tnn.lib.tnn_grid_backward(ctypes.byref(gd), ptr(x), ptr(denc), FP16, W, ptr(grad_table), 1, M, s))

    def snapshot():
        torch.cuda.synchronize()
        return [t.clone() for t in (enc, y, loss, dW, denc, grad_table)]

    step()  # eager once: kernel attributes are set, nothing is left to initialise during the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.current_stream().wait_stream(side)

    for it in range(4):
        # new inputs, written in place so that the recorded pointers stay valid
        x.copy_(torch.rand((M, 2), device=tnn.dev, generator=gen))
        targets.copy_(torch.rand((M, W), device=tnn.dev, generator=gen))
        step()
        eager = snapshot()
        for t in (enc, y, loss, dW, denc, grad_table):
            t.fill_(float("nan"))   # eager work of the program's own between the replays
        graph.replay()
        replayed = snapshot()
        for name, a, b in zip(("encoding", "y", "loss", "dW", "dL/d(encoding)", "gradient table"), eager, replayed):
            if name == "gradient table":   # float atomics: the order of additions differs from run to run
                assert torch.allclose(a, b, rtol=1e-4, atol=1e-6 * float(a.abs().max())), f"replay {it}: {name}"
            else:
                assert torch.equal(a, b), f"replay {it}: {name}"


def test_captured_fused_grid_step_replays_like_eager(tnn):
    """The same for the step that orders the batch by cell and runs encoding, network step (with Adam) and scatter as one call:
    tnn_grid_order_points + tnn_grid_mlp_train_step_l2_adam recorded once, replayed on new points and targets. The weights are
    restored before every run so that eager and replayed steps start from the same state."""
    M, n_hidden = 1 << 14, 2
    n_mats = n_hidden + 1
    gen = torch.Generator(device=tnn.dev).manual_seed(10)
    gd = tnn.grid_desc(CFG, FP16)
    g = ctypes.byref(gd)
    n_table = tnn.grid_n_params(gd)
    table = (torch.rand(n_table, device=tnn.dev, generator=gen) * 2 - 1).to(torch.float16)
    desc = tnn.mlp_desc(FP16, W, n_hidden, "relu", "none")
    d = ctypes.byref(desc)
    master0 = (torch.rand(n_mats * W * W, device=tnn.dev, generator=gen) * 2 - 1) * 0.2
    master = master0.clone()
    pf0, pb0 = tnn.prepare_packed(desc, master0, src_is_fp32=True)
    pf, pb = pf0.clone(), pb0.clone()
    m, v = torch.zeros_like(master), torch.zeros_like(master)
    x = torch.rand((M, 2), device=tnn.dev, generator=gen)
    targets = torch.rand((M, W), device=tnn.dev, generator=gen)
    y = torch.empty((M, W), dtype=torch.float16, device=tnn.dev)
    loss = torch.zeros(1, device=tnn.dev)
    grad_table = torch.empty(n_table, device=tnn.dev)
    order_bytes = tnn.lib.tnn_grid_order_bytes(g, M)
    order = torch.empty(order_bytes, dtype=torch.uint8, device=tnn.dev)
    ws_bytes = tnn.lib.tnn_grid_mlp_train_step_workspace_bytes(g, d, M)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=tnn.dev)

    def restore():
        master.copy_(master0); pf.copy_(pf0); pb.copy_(pb0); m.zero_(); v.zero_()

    def step():
        s = tnn.stream()
        _lib.check(tnn.lib.tnn_grid_order_points(g, ptr(x), M, ptr(order), order_bytes, s))
        _lib.check(tnn.lib.tnn_grid_mlp_train_step_l2_adam(g, d, None, ptr(order), ptr(table), ptr(pf), ptr(pb), ptr(targets), 4096.0, ptr(y),
                                                           ptr(loss), ptr(master), ptr(m), ptr(v), 1, 1e-2, 0.9, 0.99, 1e-8, None, ptr(grad_table), 1,
                                                           M, ptr(ws), ws_bytes, s))

    def snapshot():
        torch.cuda.synchronize()
        return [t.clone() for t in (y, loss, master, pf, pb, grad_table)]

    step()
    torch.cuda.synchronize()
    restore()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.current_stream().wait_stream(side)

    for it in range(4):
        x.copy_(torch.rand((M, 2), device=tnn.dev, generator=gen))
        targets.copy_(torch.rand((M, W), device=tnn.dev, generator=gen))
        restore()
        step()
        eager = snapshot()
        restore()
        for t in (y, loss, grad_table):
            t.fill_(float("nan"))
        graph.replay()
        replayed = snapshot()
        # Per-row results are bit-equal. Points of one cell take their places in the cell order by LDS atomics, so two runs put
        # other rows into a tile and take the fp32 sums over the batch (loss, weight gradients, table gradients) in another
        # order: those, and what Adam makes of them, agree to rounding.
        for name, a, b in zip(("y", "loss", "master", "forward weights", "backward weights", "gradient table"), eager, replayed):
            if name == "y":
                assert torch.equal(a, b), f"replay {it}: {name}"
            elif name == "loss":
                assert abs(float(a) - float(b)) <= 1e-5 * abs(float(a)), f"replay {it}: {name}"
            elif name == "master":
                assert torch.allclose(a, b, rtol=1e-5, atol=2e-6), f"replay {it}: {name}: {float((a - b).abs().max())}"
            elif name == "gradient table":
                assert torch.allclose(a, b, rtol=1e-4, atol=1e-6 * float(a.abs().max())), f"replay {it}: {name}"
            else:
                assert torch.allclose(a.float(), b.float(), rtol=2 ** -7, atol=1e-5), f"replay {it}: {name}"
                assert float((a.view(torch.int16) != b.view(torch.int16)).float().mean()) < 0.01, f"replay {it}: {name}: too many weights rounded the other way"
        assert float(eager[1]) > 0
