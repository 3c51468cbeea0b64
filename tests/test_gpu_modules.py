"""GPU tests of the Python package (tiny_dpcpp_nn.Network / Encoding / NetworkWithInputEncoding).

They follow the reference's Python tests: forward and gradients against an fp32 linear stack built from the same
weights (test/python/test_compare_torch_dpcpp.py:92-157,185-242), set/get params (test_set_param.py:48-61),
zeroed padding weights (test_padding_bias.py:176-213), output shapes of encodings (test_encodings.py:607-608), and
a short training run (test_training.py). Network results are also checked against the CPU oracle, which rounds
where the kernels round.

Tolerances: tests/tolerances.py (bf16 1e-2 rel / 1e-3 abs, fp16 5e-3 rel / 5e-4 abs; end to end "propagated").
"""
import numpy as np
import pytest
import torch

from oracle_bindings import BF16, FP16
from tolerances import assert_propagated, max_norm_rel

pytestmark = pytest.mark.gpu

DEVICE = "cuda"
DT = {torch.float16: FP16, torch.bfloat16: BF16}


@pytest.fixture(scope="module")
def tcnn():
    import tiny_dpcpp_nn

    assert torch.cuda.is_available(), "these tests need the GPU"
    return tiny_dpcpp_nn


@pytest.fixture(autouse=True)
def same_networks_every_run(tcnn):
    """A network's initial weights are seeded from std::random_device, as the reference's are; comparisons near their tolerance
    would then pass in one run and fail in the next. Every test starts from the same seed instead."""
    tcnn.manual_seed(20240607)


def net_config(width, n_hidden, act="relu", out_act="none"):
    return {"otype": "FullyFusedMLP", "activation": act, "output_activation": out_act, "n_neurons": width, "n_hidden_layers": n_hidden}


def packed_index(width):
    """perm[k * W + n] = position of element (k=in, n=out) inside one packed matrix."""
    k, n = np.divmod(np.arange(width * width), width)
    return (k & ~1) * width + 2 * n + (k & 1)


def unpack(packed, n_mats, width):
    """Packed parameter vector -> (n_mats, W, W) array indexed [matrix][in][out]."""
    p = np.asarray(packed, np.float32).reshape(n_mats, width * width)
    return p[:, packed_index(width)].reshape(n_mats, width, width)


def random_weights(n_mats, width, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    bound = (6.0 / (2 * width)) ** 0.5
    w = (torch.rand(n_mats, width, width, generator=g) * 2 - 1) * bound
    return w.to(dtype).to(torch.float32)  # values representable in dtype


def torch_reference(x_padded, weights, act, out_act):
    """fp32 autograd reference: y = f_out(f(...f(x W_0)...) W_L) with [in][out] matrices."""
    fns = {"relu": torch.relu, "sigmoid": torch.sigmoid, "none": lambda t: t}
    h = x_padded
    for i, w in enumerate(weights):
        h = h @ w
        h = fns[out_act if i == len(weights) - 1 else act](h)
    return h


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("width,n_hidden,n_in,n_out,act,out_act,use_bias,batch", [
    (64, 4, 64, 64, "relu", "none", False, 1024),
    (64, 2, 32, 3, "relu", "none", True, 512),
    (16, 2, 16, 16, "sigmoid", "none", False, 64),
    (32, 3, 5, 7, "none", "sigmoid", True, 13),       # ragged batch: padded to 16 rows inside
    (128, 2, 100, 128, "relu", "relu", False, 40),
])
def test_network_forward_and_gradients(tcnn, oracle, dtype, width, n_hidden, n_in, n_out, act, out_act, use_bias, batch):
    torch.manual_seed(0)
    n_mats = n_hidden + 1
    net = tcnn.Network(n_in, n_out, net_config(width, n_hidden, act, out_act), dtype=dtype, use_bias=use_bias)
    assert net.params.dtype == torch.float32 and net.params.numel() == n_mats * width * width
    assert net.loss_scale == (128.0 if dtype == torch.float16 else 1.0)

    w = random_weights(n_mats, width, 42, dtype)
    net.set_params(w.reshape(-1).to(DEVICE))

    # what the module holds: packed; rows of W_0 beyond the one-padded input width and columns of W_L beyond n_out are zero
    # (include/network/Network.h:182-203 of the reference: with use_bias an input width that already is a multiple of 16
    # keeps every row, the ones the module pads with then reach all of them)
    one_padded = n_in if not use_bias else (width if n_in % 16 == 0 else ((n_in + 15) // 16) * 16)
    w_eff = w.clone()
    w_eff[0, one_padded:, :] = 0
    w_eff[-1, :, n_out:] = 0
    held = unpack(net.get_params().float().cpu().numpy().reshape(-1), n_mats, width)
    np.testing.assert_array_equal(held, w_eff.numpy())
    np.testing.assert_array_equal(unpack(net.params.detach().cpu().numpy().reshape(-1), n_mats, width), w_eff.numpy())

    x = (torch.rand(batch, n_in) * 2 - 1).to(dtype)
    x_dev = x.to(DEVICE).requires_grad_(True)
    x_pad = torch.nn.functional.pad(x.float(), [0, width - n_in], value=float(use_bias))

    # ---- eval mode: the inference kernel
    net.eval()
    with torch.no_grad():
        y_eval = net(x_dev)
    assert y_eval.shape == (batch, n_out) and y_eval.dtype == dtype
    n_rows = ((batch + 7) // 8) * 8
    x_or = np.zeros((n_rows, width), np.float32)
    x_or[:batch] = x_pad.numpy()
    interm = oracle.mlp_forward_T(DT[dtype], width, n_mats, act, out_act, w_eff.numpy(), x_or)
    y_oracle = interm[-1][:batch, :n_out]
    assert_propagated(y_eval.float().cpu().numpy(), y_oracle, DT[dtype], "inference vs oracle")

    # ---- train mode: forward that keeps activations, then backward through autograd
    net.train()
    y = net(x_dev)
    assert y.shape == (batch, n_out)
    np.testing.assert_array_equal(y.detach().float().cpu().numpy(), y_eval.float().cpu().numpy())
    g = ((torch.rand(batch, n_out) * 2 - 1) / batch).to(dtype)
    y.backward(g.to(DEVICE))

    ws = [w_eff[i].clone().requires_grad_(True) for i in range(n_mats)]
    x_ref = x_pad.clone().requires_grad_(True)
    y_ref = torch_reference(x_ref, ws, act, out_act)
    assert max_norm_rel(y.detach().float().cpu().numpy(), y_ref[:, :n_out].detach().numpy()) <= 1e-2
    y_ref[:, :n_out].backward(g.float())

    # parameter gradients arrive in the parameter (packed) layout and in the parameter dtype
    assert net.params.grad is not None and net.params.grad.shape == net.params.shape and net.params.grad.dtype == torch.float32
    dW = unpack(net.params.grad.cpu().numpy().reshape(-1), n_mats, width)
    assert x_dev.grad is not None and x_dev.grad.shape == (batch, n_in)
    dx = x_dev.grad.float().cpu().numpy()

    # (1) against the oracle, which rounds where the kernels round: it gets the loss-scaled dL/dy the module hands to
    # the kernels, its results are divided by the loss scale as the module does
    g_or = np.zeros((n_rows, width), np.float32)
    g_or[:batch, :n_out] = (g * net.loss_scale).float().numpy()
    _, dW_or, dX_or = oracle.mlp_backward_T(DT[dtype], width, n_mats, act, out_act, w_eff.numpy(), interm, g_or)
    dW_or = dW_or.transpose(0, 2, 1) / net.loss_scale       # [out][in] -> [in][out]
    dX_or = dX_or[:batch, :n_in] / net.loss_scale
    assert_propagated(dW, dW_or, DT[dtype], "dW vs oracle", scale=float(np.abs(dW_or).max()))
    assert_propagated(dx, dX_or, DT[dtype], "dL/dx vs oracle", scale=float(np.abs(dX_or).max()))

    # (2) against fp32 autograd, as the reference's Python tests compare (test_compare_torch_dpcpp.py:185-242). The fp32
    # chain does not round between layers, so a pre-activation within rounding distance of zero can get the other ReLU
    # mask and move single gradient entries by one sample's worth (a tenth of the largest entry at batch 40); the
    # check is therefore on the whole gradient: relative error in the Frobenius norm, 4e-2 for fp16 and 1e-1 for bf16
    # (8 significant bits at each of the roundings on the way; measured 2.5e-2 and 6.5e-2 for dL/dx through five ReLU
    # layers, where a flipped mask is not averaged over the batch). A wrong layout or scale gives an error of order 1.
    dW_ref = np.stack([wi.grad.numpy() for wi in ws])
    dx_ref = x_ref.grad[:, :n_in].numpy()
    bar = 4e-2 if dtype == torch.float16 else 1e-1
    for got, ref, what in ((dW, dW_ref, "dW"), (dx, dx_ref, "dL/dx")):
        err = np.linalg.norm((got - ref).ravel()) / np.linalg.norm(ref.ravel())
        assert err <= bar, f"{what}: relative Frobenius error {err:g} vs fp32 autograd"

    # an input that asks for no gradient: the backward leaves dL/dinput out, the parameter gradient is the same
    grad_with_dx = net.params.grad.clone()
    net.params.grad = None
    net(x.to(DEVICE)).backward(g.to(DEVICE))
    assert torch.equal(net.params.grad, grad_with_dx)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_set_params_constant(tcnn, dtype):
    """test_set_param.py:24-70 of the reference."""
    width = 16
    net = tcnn.Network(16, 16, net_config(width, 3, "None", "None"), dtype=dtype)
    x = (torch.ones(8, width) * 0.1).to(DEVICE, dtype=dtype)
    param_vals = 0.123 * torch.ones(width * width * 4, 1, dtype=dtype).to(DEVICE)
    net.set_params(param_vals)
    assert torch.isclose(param_vals, net.params.to(dtype)).all()
    assert torch.isclose(param_vals, net.params.data.to(dtype)).all()
    y = net(x)
    assert torch.isfinite(y).all()
    # closed form: every layer multiplies by 16 * w (activation None)
    w = float(torch.tensor(0.123, dtype=dtype))
    expect = 0.1 * (16 * w) ** 4
    assert torch.allclose(y.float(), torch.full_like(y.float(), expect), rtol=2e-2)


@pytest.mark.parametrize("n_neurons", [16, 32, 64, 128])
@pytest.mark.parametrize("n_hidden_layers", [1, 2, 4])
def test_padding_weights_are_zero(tcnn, n_neurons, n_hidden_layers):
    """test_padding_bias.py:176-213 of the reference: freshly initialised weights that only see padding are zero."""
    n_in, n_out = 3, 5
    net = tcnn.Network(n_in, n_out, net_config(n_neurons, n_hidden_layers, "none", "none"))
    mats = unpack(net.get_params().float().cpu().numpy().reshape(-1), n_hidden_layers + 1, n_neurons)
    assert np.all(mats[0][16:, :] == 0)       # use_bias=True: the input is padded with ones up to 16, zeros beyond
    assert np.any(mats[0][:16, :] != 0)
    assert np.all(mats[-1][:, n_out:] == 0)
    assert np.any(mats[-1][:, :n_out] != 0)
    # Xavier bound of the reference: +-sqrt(6 / (16 + width)) for the first and the last matrix, +-sqrt(6 / (2 width)) between
    assert np.abs(mats[0]).max() <= (6.0 / (16 + n_neurons)) ** 0.5 * 1.01
    for m in mats[1:-1]:
        assert np.abs(m).max() <= (6.0 / (2 * n_neurons)) ** 0.5 * 1.01
    # padded outputs of a network without output activation are exactly zero, whatever the input
    x = torch.rand(24, n_in, device=DEVICE)
    y_full = net.tnn_module.inference(torch.nn.functional.pad(x, [0, n_neurons - n_in], value=1.0).to(torch.float16).contiguous())
    assert y_full.shape == (24, n_neurons) and torch.all(y_full[:, n_out:] == 0)


def test_network_errors(tcnn):
    with pytest.raises(RuntimeError, match="m_activation must be"):
        tcnn.Network(16, 16, net_config(16, 2, "tanh", "none"))
    with pytest.raises(NotImplementedError):
        tcnn.Network(16, 16, net_config(16, 2, "swish", "none"))
    with pytest.raises(AssertionError):
        tcnn.Network(16, 16, net_config(16, 2), dtype=torch.float32)
    with pytest.raises(RuntimeError, match="Unsupported width"):
        tcnn.Network(16, 16, net_config(48, 2))
    with pytest.raises(RuntimeError, match="not supported"):
        tcnn.Network(65, 16, net_config(64, 2))
    net = tcnn.Network(16, 16, net_config(16, 2))
    with pytest.raises(RuntimeError, match="does not match"):
        net.set_params(torch.zeros(5, device=DEVICE))
    with pytest.raises((RuntimeError, ValueError), match="divisible by 8"):
        net.tnn_module.inference(torch.zeros(7, 16, device=DEVICE, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="must be a GPU tensor"):
        net.tnn_module.inference(torch.zeros(8, 16, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="takes no input_from_fwd"):
        net.tnn_module.bwd_with_encoding_grad(torch.zeros(8, 16, device=DEVICE, dtype=torch.float16),
                                              torch.zeros(8, 16, device=DEVICE, dtype=torch.float16), False, False)
    # empty batch keeps its shape
    y = net(torch.zeros(0, 16, device=DEVICE))
    assert y.shape == (0, 16)
    tcnn.free_temporary_memory()


GRID_2D = {"otype": "HashGrid", "type": "Hash", "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 15,
           "base_resolution": 16, "per_level_scale": 1.5}
GRID_3D = {"otype": "HashGrid", "n_levels": 8, "n_features_per_level": 4, "log2_hashmap_size": 12, "base_resolution": 4,
           "per_level_scale": 2.0, "interpolation": "Linear", "hash": "CoherentPrime"}


def oracle_cfg(cfg, n_dims):
    return {"n_dims": n_dims, "n_levels": cfg["n_levels"], "n_features_per_level": cfg["n_features_per_level"],
            "log2_hashmap_size": cfg["log2_hashmap_size"], "base_resolution": cfg["base_resolution"],
            "per_level_scale": cfg["per_level_scale"], "grid_type": cfg.get("type", "Hash"),
            "hash": cfg.get("hash", "CoherentPrime"), "interpolation": cfg.get("interpolation", "Linear")}


@pytest.mark.parametrize("cfg,n_dims,padded,batch", [(GRID_2D, 2, None, 1000), (GRID_2D, 2, 64, 256), (GRID_3D, 3, 64, 777)])
def test_encoding_forward_and_gradients(tcnn, oracle, cfg, n_dims, padded, batch):
    enc = tcnn.Encoding(n_dims, dict(cfg), n_output_dims=padded)
    n_feat = cfg["n_levels"] * cfg["n_features_per_level"]
    width = padded if padded is not None else n_feat
    assert enc.n_output_dims == width
    assert enc.params.dtype == torch.float32 and enc.params.requires_grad
    init = enc.params.detach().cpu().numpy()
    assert np.abs(init).max() <= 1e-4 and abs(init.mean()) < 1e-5 and init.std() > 3e-5   # uniform in +-1e-4

    torch.manual_seed(3)
    table = (torch.rand(enc.params.numel(), device=DEVICE) * 2 - 1)
    enc.set_params(table)
    np.testing.assert_array_equal(enc.get_params().cpu().numpy().reshape(-1), table.cpu().numpy())
    np.testing.assert_array_equal(enc.params.detach().cpu().numpy().reshape(-1), table.cpu().numpy())

    x = torch.rand(batch, n_dims)
    x[0] = 0.0
    x[1] = 1.0
    y = enc(x.to(DEVICE))
    assert y.shape == (batch, width) and y.dtype == torch.float32
    ocfg = oracle_cfg(cfg, n_dims)
    y_ref = oracle.grid_forward(ocfg, table.cpu().numpy(), x.numpy(), width)
    np.testing.assert_allclose(y.detach().cpu().numpy(), y_ref, rtol=0, atol=2e-6)
    if width > n_feat:
        assert torch.all(y[:, n_feat:] == 0)

    g = torch.rand(batch, width) * 2 - 1
    y.backward(g.to(DEVICE))
    grad = enc.params.grad.cpu().numpy().reshape(-1)
    grad_ref = oracle.grid_backward(ocfg, x.numpy(), g.numpy(), table.numel())
    assert max_norm_rel(grad, grad_ref) <= 1e-5


def test_encoding_errors(tcnn):
    with pytest.raises((RuntimeError, ValueError), match="Unknown encoding type"):
        tcnn.Encoding(2, {"otype": "Nope"})
    with pytest.raises(AssertionError):
        tcnn.Encoding(2, dict(GRID_2D), dtype=torch.float16)
    with pytest.raises((RuntimeError, ValueError), match="2 or 3"):
        tcnn.Encoding(4, dict(GRID_2D))
    enc = tcnn.Encoding(2, dict(GRID_2D))
    with pytest.raises(RuntimeError, match="incorrect dimensions"):
        enc.tnn_module.fwd(torch.zeros(8, 3, device=DEVICE))
    with pytest.raises(RuntimeError, match="needs input_from_fwd"):
        enc.tnn_module.bwd_no_encoding_grad(torch.zeros(8, 32, device=DEVICE), False, False)
    with pytest.raises((RuntimeError, ValueError), match="not packed"):
        enc.tnn_module.bwd_with_encoding_grad(torch.zeros(8, 32, device=DEVICE), torch.zeros(8, 2, device=DEVICE), True, False)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_network_with_input_encoding_trains(tcnn, dtype):
    """BASELINE-style pipeline (2-D hash grid -> 64-wide MLP, 3 outputs) learning a smooth image with torch.optim.Adam."""
    torch.manual_seed(1)
    model = tcnn.NetworkWithInputEncoding(2, 3, net_config(64, 2), dict(GRID_2D), dtype=dtype, use_bias=False)
    assert model.params is model.network.params
    assert model.encoding.n_output_dims == 64
    opt = torch.optim.Adam(model.parameters(), lr=1e-2, betas=(0.9, 0.99), eps=1e-15)
    assert sum(p.numel() for p in model.parameters()) == model.network.params.numel() + model.encoding.params.numel()

    def target(xy):
        return torch.stack([torch.sin(6 * xy[:, 0]) * 0.5 + 0.5, xy[:, 1], xy[:, 0] * xy[:, 1]], dim=1)

    losses = []
    for step in range(60):
        xy = torch.rand(4096, 2, device=DEVICE)
        out = model(xy)
        assert out.shape == (4096, 3) and out.dtype == dtype
        loss = ((out.float() - target(xy)) ** 2).mean()
        opt.zero_grad()
        loss.backward()
        assert model.network.params.grad is not None and model.encoding.params.grad is not None
        assert torch.isfinite(model.network.params.grad).all() and torch.isfinite(model.encoding.params.grad).all()
        opt.step()
        losses.append(float(loss.detach()))
    assert losses[-1] < 0.25 * losses[0], losses[::10]

    model.eval()
    with torch.no_grad():
        xy = torch.rand(1001, 2, device=DEVICE)
        out = model(xy)
    assert out.shape == (1001, 3)
    assert float(((out.float() - target(xy)) ** 2).mean()) < 0.5 * losses[0]
    with pytest.raises(RuntimeError, match="Not implemented"):
        model.get_params()


@pytest.mark.parametrize("dtype,width,n_hidden,act,out_act,batch", [
    (torch.bfloat16, 64, 4, "relu", "none", 4096), (torch.float16, 64, 2, "relu", "sigmoid", 1000), (torch.float16, 32, 3, "sigmoid", "none", 520),
    (torch.bfloat16, 16, 5, "relu", "relu", 8)])
def test_training_without_stored_activations_equals_the_stored_route(tcnn, dtype, width, n_hidden, act, out_act, batch):
    """A network whose shape has the one-kernel backward pass trains without stored activations: inference() forward,
    bwd_recompute() backward. Against the reference's route on the same native module (fwd() keeps every activation,
    bwd_no_encoding_grad() reads them): the output and dL/dx bit for bit, the weight gradients -- sums over the batch, rounded
    to the network's type, taken in another order -- to a unit in the last place."""
    torch.manual_seed(batch)
    net = tcnn.Network(width, width, net_config(width, n_hidden, act, out_act), dtype=dtype, use_bias=False)
    native = net.tnn_module
    assert native.can_recompute_backward()
    x = (torch.rand((batch, width), device=DEVICE) * 2 - 1).to(dtype)
    dy = ((torch.rand((batch, width), device=DEVICE) * 2 - 1) * 0.1).to(dtype)
    y_stored = native.fwd(x)
    dx_stored, dw_stored = native.bwd_no_encoding_grad(dy, True, True)
    y = native.inference(x)
    dx, dw = native.bwd_recompute(dy, x, True, True)
    assert torch.equal(y.view(torch.int16), y_stored.view(torch.int16))
    assert torch.equal(dx.view(torch.int16), dx_stored.view(torch.int16))
    scale = float(dw_stored.float().abs().max())
    assert torch.allclose(dw.float(), dw_stored.float(), rtol=2 ** -7 if dtype == torch.bfloat16 else 2 ** -10, atol=1e-4 * scale)
    assert float((dw.view(torch.int16) != dw_stored.view(torch.int16)).float().mean()) < 0.02
    _, dw_only = native.bwd_recompute(dy, x, True, False)
    assert torch.equal(dw_only.view(torch.int16), dw.view(torch.int16))
    # the module takes that route by itself, in training and in evaluation mode, and two forward passes may precede their
    # backward passes (nothing of a forward pass is kept in the module)
    net.train()
    xa, xb = x[: batch // 2 + 4].float().requires_grad_(True), x.float().requires_grad_(True)
    ya, yb = net(xa), net(xb)
    (ya.float().square().mean() + yb.float().square().mean()).backward()
    assert xa.grad is not None and xb.grad is not None and net.params.grad is not None and torch.isfinite(net.params.grad).all()
    wide = tcnn.Network(128, 128, net_config(128, 2), dtype=torch.float16)
    assert not wide.tnn_module.can_recompute_backward()
    with pytest.raises(Exception, match="not available|no fused training kernel"):
        wide.tnn_module.bwd_recompute(torch.zeros((8, 128), dtype=torch.float16, device=DEVICE), torch.zeros((8, 128), dtype=torch.float16, device=DEVICE), True, False)


@pytest.mark.parametrize("dtype,n_dims,grid,n_hidden,batch", [
    (torch.float16, 2, GRID_2D, 2, 4096), (torch.bfloat16, 2, GRID_2D, 1, 1001),
    (torch.float16, 3, {"otype": "HashGrid", "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 14, "base_resolution": 16, "per_level_scale": 1.447}, 3, 2048)])
def test_network_with_grid_encoding_trains_through_one_kernel(tcnn, oracle, dtype, n_dims, grid, n_hidden, batch):
    """NetworkWithInputEncoding with autograd on a grid encoding: forward is the fused inference kernel, backward one kernel
    that forms encoding and activations again plus the scatter. Against the two modules in turn (the reference's only route,
    dpcpp_bindings/tiny_dpcpp_nn/modules.py:389-407) on the same model: output bit for bit, network gradients to a unit in the
    last place of the network's type, table gradients to 1e-5 of their largest; and against the oracle's chain."""
    torch.manual_seed(17)
    model = tcnn.NetworkWithInputEncoding(n_dims, 3, net_config(64, n_hidden), dict(grid), dtype=dtype, use_bias=False)
    with torch.no_grad():
        model.encoding.params.copy_(torch.rand_like(model.encoding.params) * 2 - 1)
    model.train()
    assert model.network.tnn_module.can_train_with_encoding(model.encoding.tnn_module)
    x = torch.rand((batch, n_dims), device=DEVICE)
    target = torch.rand((batch, 3), device=DEVICE)

    def grads(run):
        model.zero_grad(set_to_none=True)
        out = run(x)
        ((out.float() - target) ** 2).mean().backward()
        return out.detach(), model.network.params.grad.clone(), model.encoding.params.grad.clone()

    y2, dnet2, dtab2 = grads(model.network_with_encoding)   # Encoding.forward, then Network.forward
    y1, dnet1, dtab1 = grads(model)                        # one kernel each way
    assert y1.shape == (batch, 3) and y1.dtype == dtype
    assert torch.equal(y1.view(torch.int16), y2.view(torch.int16))
    net_scale, tab_scale = float(dnet2.abs().max()), float(dtab2.abs().max())
    assert net_scale > 0 and tab_scale > 0
    assert torch.allclose(dnet1, dnet2, rtol=2 ** -7 if dtype == torch.bfloat16 else 2 ** -10, atol=1e-4 * net_scale), float((dnet1 - dnet2).abs().max()) / net_scale
    # bf16 (loss scale 1): the same dL/d(encoding) bits go into the scatter on both routes, only the order of the atomic
    # additions differs. fp16 (loss scale 128): the two-module route divides dL/d(encoding) by the loss scale in fp16 before
    # the scatter, which pushes it into the subnormal range and costs it bits (about 1e-3 of the largest gradient here);
    # the fused route scatters the scaled values and divides the fp32 sums, which is the more accurate of the two -- the
    # oracle's chain below is the judge of both.
    assert float((dtab1 - dtab2).abs().max()) <= (2e-3 if dtype == torch.float16 else 1e-5) * tab_scale, float((dtab1 - dtab2).abs().max()) / tab_scale
    # the oracle's chain: encoding (fp32 table) rounded to the network's type, network forward, backward with dL/d(encoding), scatter
    W, n_mats = 64, n_hidden + 1
    T = DT[dtype]
    cfg = oracle_cfg(grid, n_dims)
    table = model.encoding.params.detach().cpu().numpy().reshape(-1)
    w = oracle.round(unpack(model.network.get_params().float().cpu().numpy().reshape(-1), n_mats, W), T)
    enc = oracle.round(oracle.grid_forward(cfg, table, x.cpu().numpy(), W), T)
    interm = oracle.mlp_forward_T(T, W, n_mats, "relu", "none", w, enc)
    assert_propagated(y1.float().cpu().numpy(), interm[-1][:, :3], T, "fused output against the oracle chain")
    scale = model.network.loss_scale
    dy = np.zeros((batch, W), np.float32)
    dy[:, :3] = (2.0 / (3 * batch)) * (y1.float().cpu().numpy() - target.cpu().numpy()) * scale
    dy = oracle.round(dy, T)
    _, rdW, rd_enc = oracle.mlp_backward_T(T, W, n_mats, "relu", "none", w, interm, dy, round_dw=False)
    ref_tab = oracle.grid_backward(cfg, x.cpu().numpy(), rd_enc, table.size) / scale
    assert max_norm_rel(dtab1.cpu().numpy().reshape(-1), ref_tab) <= (1e-2 if dtype == torch.bfloat16 else 5e-3)
    # rdW is raw [out][in]; the module's gradient is packed [in][out]
    got = unpack(dnet1.float().cpu().numpy().reshape(-1), n_mats, W)
    assert max(max_norm_rel(got[l], rdW[l].T / scale) for l in range(n_mats)) <= (1e-2 if dtype == torch.bfloat16 else 5e-3)
    # evaluation mode with autograd takes the same route; positions get no gradient
    model.eval()
    xg = x.clone().requires_grad_(True)
    model(xg).float().sum().backward()
    assert xg.grad is None


def test_fused_training_route_at_a_batch_that_is_visited_in_cell_order(tcnn):
    """From 2^17 rows on the fused backward pass visits the points in cell order (its tiles then hold other rows than the batch's,
    and the order differs from run to run): sums over the batch agree with the two-module route to fp32 rounding, the per-row
    output bit for bit. BASELINE config 4's shapes (2-D, 16 x 2, log2 19, w64 with 2 hidden layers, 3 outputs), half its batch."""
    torch.manual_seed(23)
    grid = {"otype": "HashGrid", "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 19, "base_resolution": 16, "per_level_scale": 1.5}
    model = tcnn.NetworkWithInputEncoding(2, 3, net_config(64, 2), grid, dtype=torch.float16, use_bias=False)
    with torch.no_grad():
        model.encoding.params.copy_(torch.rand_like(model.encoding.params) * 2 - 1)
    model.train()
    batch = (1 << 17) + 8
    x = torch.rand((batch, 2), device=DEVICE)
    target = torch.rand((batch, 3), device=DEVICE)

    def grads(run):
        model.zero_grad(set_to_none=True)
        out = run(x)
        ((out.float() - target) ** 2).mean().backward()
        return out.detach(), model.network.params.grad.clone(), model.encoding.params.grad.clone()

    y2, dnet2, dtab2 = grads(model.network_with_encoding)
    y1, dnet1, dtab1 = grads(model)
    assert torch.equal(y1.view(torch.int16), y2.view(torch.int16))
    net_scale, tab_scale = float(dnet2.abs().max()), float(dtab2.abs().max())
    assert torch.allclose(dnet1, dnet2, rtol=2 ** -9, atol=2e-4 * net_scale), float((dnet1 - dnet2).abs().max()) / net_scale
    # (the two-module route divides dL/d(encoding) by the loss scale in fp16, which at this batch size lies deep in the
    # subnormal range and keeps few bits; the fused route divides the fp32 sums -- see the test above, where the oracle judges)
    assert float((dtab1 - dtab2).abs().max()) <= 1e-2 * tab_scale, float((dtab1 - dtab2).abs().max()) / tab_scale
    assert float(dtab1.abs().sum()) > 0 and torch.isfinite(dtab1).all()
    # the same model in bf16 has loss scale 1: the same dL/d(encoding) bits reach the scatter on both routes
    model16 = tcnn.NetworkWithInputEncoding(2, 3, net_config(64, 2), grid, dtype=torch.bfloat16, use_bias=False)
    with torch.no_grad():
        model16.encoding.params.copy_(model.encoding.params)
    model16.train()

    def grads16(run):
        model16.zero_grad(set_to_none=True)
        ((run(x).float() - target) ** 2).mean().backward()
        return model16.encoding.params.grad.clone()

    ta, tb_ = grads16(model16.network_with_encoding), grads16(model16)
    assert float((ta - tb_).abs().max()) <= 1e-5 * float(ta.abs().max())


def test_backward_takes_over_the_forward_pass_cell_order_only_when_it_is_that_batch_s(tcnn):
    """The fused forward pass of a training step orders a large batch by cell and the backward pass uses that order again
    instead of forming it a second time; the native module keeps one order, the last one formed. Two forward passes on
    different batches followed by the backward pass of the FIRST must therefore order the first batch again (its order is no
    longer the one kept); the backward pass of the second then finds its own order gone as well. Gradients of both must be
    what each batch gives on its own."""
    torch.manual_seed(31)
    grid = {"otype": "HashGrid", "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 19, "base_resolution": 16, "per_level_scale": 1.5}
    model = tcnn.NetworkWithInputEncoding(2, 3, net_config(64, 2), grid, dtype=torch.bfloat16, use_bias=False)
    with torch.no_grad():
        model.encoding.params.copy_(torch.rand_like(model.encoding.params) * 2 - 1)
    model.train()
    batch = 1 << 17
    xa, xb = torch.rand((batch, 2), device=DEVICE), torch.rand((batch, 2), device=DEVICE)
    ta, tb = torch.rand((batch, 3), device=DEVICE), torch.rand((batch, 3), device=DEVICE)

    def alone(x, t):
        model.zero_grad(set_to_none=True)
        ((model(x).float() - t) ** 2).mean().backward()  # forward orders, backward takes the order over
        return model.network.params.grad.clone(), model.encoding.params.grad.clone()

    na, ea = alone(xa, ta)
    nb, eb = alone(xb, tb)
    model.zero_grad(set_to_none=True)
    la = ((model(xa).float() - ta) ** 2).mean()
    lb = ((model(xb).float() - tb) ** 2).mean()  # the order kept is now xb's
    la.backward()  # must not scatter xa's gradients over xb's order
    n1, e1 = model.network.params.grad.clone(), model.encoding.params.grad.clone()
    model.zero_grad(set_to_none=True)
    lb.backward()  # and the order kept is xa's again
    n2, e2 = model.network.params.grad.clone(), model.encoding.params.grad.clone()
    for got, want in ((n1, na), (e1, ea), (n2, nb), (e2, eb)):
        scale = float(want.abs().max())
        assert scale > 0
        assert float((got - want).abs().max()) <= 1e-4 * scale, float((got - want).abs().max()) / scale
    # a batch written to in place after its forward pass: autograd refuses the backward pass (which is what lets it reuse the order)
    model.zero_grad(set_to_none=True)
    xc = xa.clone()
    lc = ((model(xc).float() - ta) ** 2).mean()
    xc.mul_(0.5)
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        lc.backward()


def test_manual_seed_makes_initial_weights_reproducible(tcnn):
    """Two networks created after the same manual_seed hold the same weights; the next network of a sequence and a network
    created without a fixed seed (the reference's behaviour, std::random_device) hold others."""
    tcnn.manual_seed(7)
    a = tcnn.Network(32, 16, net_config(64, 2), dtype=torch.bfloat16)
    b = tcnn.Network(32, 16, net_config(64, 2), dtype=torch.bfloat16)
    tcnn.manual_seed(7)
    c = tcnn.Network(32, 16, net_config(64, 2), dtype=torch.bfloat16)
    assert torch.equal(a.params, c.params)
    assert not torch.equal(a.params, b.params)
    assert float(a.params.detach().abs().max()) > 0


def test_parameter_free_encodings_through_the_package(tcnn, oracle):
    """test/python/test_encodings.py:377-630 of the reference: spherical harmonics (golden rows), identity, padding, frequency."""
    import json
    import math
    import os

    ones = torch.ones((10, 3), device=DEVICE)
    sh = tcnn.Encoding(n_input_dims=3, encoding_config={"otype": "SphericalHarmonics", "degree": 4})
    assert sh.n_output_dims == 16 and not sh.params.requires_grad
    fx = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "spherical_harmonics_degree4.json")))
    out = sh(ones)
    assert out.shape == (10, 16) and out.dtype == torch.float32
    assert torch.all(torch.isclose(out.cpu(), torch.tensor(fx["expected_row"]).expand(10, 16), atol=fx["atol"]))

    ident = tcnn.Encoding(n_input_dims=3, encoding_config={"otype": "Identity", "scale": 1.0, "offset": 0.0})
    assert torch.all(torch.isclose(ident(ones), ones))
    wide = tcnn.Encoding(n_input_dims=3, encoding_config={"otype": "Identity", "scale": 1.0, "offset": 0.0}, n_output_dims=5346)
    y = wide(torch.rand((13, 3), device=DEVICE))            # a batch that is not a multiple of 8
    assert wide.n_output_dims == 5346 and y.shape == (13, 5346) and bool((y[:, 3:] == 1).all())

    freq = tcnn.Encoding(n_input_dims=1, encoding_config={"otype": "Frequency", "n_frequencies": 1.0})
    v = 1.234
    out = freq(torch.ones(1, 1, device=DEVICE) * v)
    assert torch.allclose(out.cpu(), torch.tensor([[math.sin(math.pi * v), math.cos(math.pi * v)]]), atol=1e-4)

    x = torch.rand((100, 3), device=DEVICE)
    f2 = tcnn.Encoding(n_input_dims=3, encoding_config={"otype": "Frequency", "n_frequencies": 4}, n_output_dims=32)
    np.testing.assert_allclose(f2(x).cpu().numpy(), oracle.frequency_forward(x.cpu().numpy(), 4, 32), atol=2e-6)
    with pytest.raises((RuntimeError, ValueError), match="Config misses"):
        tcnn.Encoding(n_input_dims=3, encoding_config={"otype": "Identity", "scale": 1.0})
    with pytest.raises(RuntimeError, match="Network has no parameters"):
        ident.set_params(torch.zeros(3, device=DEVICE))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n_dims, grid, batch", [(2, "GRID_2D", 1001), (3, "GRID_3D", 4096)])
def test_network_with_grid_encoding_fused_inference(tcnn, dtype, n_dims, grid, batch):
    """Evaluation without autograd takes the single-kernel route (encoding + network); with autograd enabled the two
    modules run in turn. Same bits either way, also for a batch that is padded to a multiple of 8."""
    cfg = dict(GRID_2D) if grid == "GRID_2D" else {"otype": "HashGrid", "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 15,
                                                   "base_resolution": 16, "per_level_scale": 1.447}
    torch.manual_seed(3)
    model = tcnn.NetworkWithInputEncoding(n_dims, 5, net_config(64, 3), cfg, dtype=dtype, use_bias=False)
    with torch.no_grad():
        model.encoding.params.copy_(torch.rand_like(model.encoding.params) * 2 - 1)  # the initial table is +-1e-4
    model.eval()
    assert model.network.tnn_module.can_fuse_encoding(model.encoding.tnn_module)
    x = torch.rand((batch, n_dims), device=DEVICE)
    two_calls = model(x).detach()  # autograd on: Encoding.forward, then Network.forward
    with torch.no_grad():
        fused = model(x)
    assert fused.shape == two_calls.shape == (batch, 5) and fused.dtype == dtype
    assert float(two_calls.float().abs().max()) > 1e-3
    assert torch.equal(fused.view(torch.int16), two_calls.view(torch.int16))
    # an encoding without a grid, or a network whose weights do not fit LDS beside it, keeps the two calls
    sh = tcnn.NetworkWithInputEncoding(3, 3, net_config(64, 2), {"otype": "SphericalHarmonics", "degree": 4}, dtype=dtype)
    assert not sh.network.tnn_module.can_fuse_encoding(sh.encoding.tnn_module)
    with pytest.raises(Exception, match="two calls"):
        sh.network.tnn_module.inference_with_encoding(sh.encoding.tnn_module, torch.rand((8, 3), device=DEVICE))


class SimpleSGD(torch.optim.Optimizer):
    """The reference's debugging optimizer (test/python/test_training.py:28-51): it updates through `p.data`, which PyTorch's
    version counter does not see."""

    def __init__(self, params, lr):
        super().__init__(params, dict(lr=lr))

    def step(self, closure=None):
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is not None:
                    p.data.copy_(p.data - group["lr"] * p.grad.data)


def test_training_through_data_writes(tcnn):
    """The reference's SimpleSGDOptimizer loop (test/python/test_training.py:28-51, 62-140): every step writes the parameters
    through `.data`; the next forward must run on the new weights, so the loss of a linear regression target falls."""
    torch.manual_seed(5)
    width = 32
    net = tcnn.Network(width, 1, net_config(width, 2, "relu", "none"), dtype=torch.bfloat16)
    opt = SimpleSGD(net.parameters(), lr=1e-2)
    x = torch.ones((8, width), device=DEVICE)
    target = 0.5 * x[:, :1]
    net.train()
    losses, outputs = [], []
    for _ in range(40):
        y = net(x)
        loss = (y.float() - target).square().mean()
        opt.zero_grad()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
        outputs.append(y.detach().clone())
    assert not torch.equal(outputs[0], outputs[1]), "a step written through .data did not reach the kernels"
    assert losses[-1] < 0.05 * losses[0], losses


def test_params_data_assignment_reaches_the_kernels(tcnn):
    """`network.params.data[:] = ...` followed by a forward (test/python/test_padding_bias.py:169-172), in evaluation mode too."""
    torch.manual_seed(6)
    net = tcnn.Network(8, 4, net_config(32, 2, "none", "none"), dtype=torch.bfloat16, use_bias=False)
    x = torch.rand((16, 8), device=DEVICE)
    for train in (True, False):
        net.train(train)
        net.params.data[:] = 0.0
        with torch.no_grad():
            assert float(net(x).float().abs().max()) == 0.0
        net.params.data[:] = torch.full_like(net.params, 0.03125)
        with torch.no_grad():
            y = net(x)
        # every weight 1/32, no activation: column sums of x over the 8 real inputs, then 32 * (1/32) per later matrix
        expect = (x.to(torch.bfloat16).float().sum(1, keepdim=True) / 32).expand(-1, 4)
        assert torch.allclose(y.float(), expect, rtol=2e-2, atol=1e-3)
    # an encoding's table is the tensor itself (no copy is pushed): a write through .data is seen by the next forward
    enc = tcnn.Encoding(2, dict(GRID_2D))
    pts2 = torch.rand((64, 2), device=DEVICE)
    enc.params.data[:] = 0.25
    with torch.no_grad():
        e = enc(pts2)
    assert torch.allclose(e[:, :32], torch.full_like(e[:, :32], 0.25), atol=1e-6)   # the corner weights of a cell sum to one
    enc.params.data[:] = 0.0
    with torch.no_grad():
        assert float(enc(pts2).abs().max()) == 0.0
    assert float(enc.get_params().abs().max()) == 0.0 and enc.get_params().data_ptr() != enc.params.data_ptr()
    # the fused encoding + network route reads both modules' parameters the same way
    nwe = tcnn.NetworkWithInputEncoding(2, 3, net_config(64, 2), dict(GRID_2D), dtype=torch.float16)
    nwe.eval()
    pts = torch.rand((64, 2), device=DEVICE)
    with torch.no_grad():
        nwe.encoding.params.data[:] = torch.rand_like(nwe.encoding.params) * 2 - 1
        y0 = nwe(pts).clone()
        nwe.encoding.params.data[:] = 0.0
        y1 = nwe(pts)
    assert float(y0.float().abs().max()) > 0.0 and float(y1.float().abs().max()) == 0.0


def test_parameters_are_pushed_when_they_change(tcnn):
    """With push_params_every_forward switched off, forward() refreshes the native module's copy of the parameters only when
    `params` changed since the last push: an optimizer step, copy_() and a replaced Parameter are all seen; a write through
    `.data` then needs an explicit set_params(). The default pushes every time, as the reference does."""
    torch.manual_seed(11)
    net = tcnn.Network(8, 4, net_config(32, 2), dtype=torch.bfloat16)
    assert net.push_params_every_forward
    net.push_params_every_forward = False
    x = torch.rand((64, 8), device=DEVICE)
    opt = torch.optim.Adam(net.parameters(), lr=1e-2)
    net.train()
    y0 = net(x)
    y0.float().square().sum().backward()
    opt.step()
    y1 = net(x)
    assert not torch.equal(y0, y1), "the optimizer step did not reach the kernels"
    y1b = net(x)
    assert torch.equal(y1, y1b)
    state = net._pushed
    net(x)
    assert net._pushed == state, "nothing changed, nothing is pushed again"
    with torch.no_grad():
        net.params.copy_(torch.zeros_like(net.params))
    assert float(net(x).detach().float().abs().max()) == 0.0, "copy_() into params did not reach the kernels"
    net.params.data.fill_(0.01)  # invisible to the version counter
    net.set_params()
    assert float(net(x).detach().float().abs().max()) > 0.0
    net.params = torch.nn.Parameter(torch.zeros_like(net.params))
    assert float(net(x).detach().float().abs().max()) == 0.0, "a replaced Parameter did not reach the kernels"


def test_modules_follow_the_callers_stream(tcnn):
    """A module's kernels go to torch's current stream at the time of the call: an input that is still being produced on a
    side stream is complete when they read it, without any host wait, and a module can move between streams."""
    torch.manual_seed(2)
    net = tcnn.Network(64, 64, net_config(64, 2), dtype=torch.bfloat16, use_bias=False)
    enc = tcnn.Encoding(2, dict(GRID_2D))
    net.eval()
    enc.eval()
    n = 1 << 16
    base = torch.rand((n, 64), device=DEVICE)
    pos = torch.rand((n, 2), device=DEVICE)
    big = torch.rand((4096, 4096), device=DEVICE)
    with torch.no_grad():
        want = net((base * 2 - 1)), enc(pos * 0.5)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(10):
                busy = big @ big  # keeps the side stream busy while the host runs ahead
            x = base * 2 - 1 + busy[0, 0] * 0  # produced behind that work, on the side stream
            p = pos * 0.5 + busy[0, 0] * 0
            got = net(x), enc(p)
        side.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w)
        # back on the default stream the module waits for what it left on the side stream by itself
        again = net(base * 2 - 1)
        torch.cuda.synchronize()
        assert torch.equal(again, want[0])


def test_large_batches_take_the_cell_order_route(tcnn):
    """From 2^18 rows on the grid encoding (alone, and fused with the network) orders the batch by cell first. Row for row the
    result equals what the same rows give in batches below the threshold."""
    n = (1 << 19) + 40
    cfg = {"otype": "HashGrid", "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 17, "base_resolution": 16, "per_level_scale": 1.447}
    torch.manual_seed(5)
    model = tcnn.NetworkWithInputEncoding(3, 4, net_config(64, 2), cfg, dtype=torch.float16, use_bias=False)
    with torch.no_grad():
        model.encoding.params.copy_(torch.rand_like(model.encoding.params) * 2 - 1)
    model.eval()
    x = torch.rand((n, 3), device=DEVICE)
    with torch.no_grad():
        big = model(x)
        enc_big = model.encoding(x)
        for lo in (0, 250000, n - 1000):
            assert torch.equal(model(x[lo:lo + 1000]).view(torch.int16), big[lo:lo + 1000].view(torch.int16))
            assert torch.equal(model.encoding(x[lo:lo + 1000]), enc_big[lo:lo + 1000])
    assert float(big.float().abs().max()) > 1e-3


def test_large_batches_scatter_in_cell_order(tcnn):
    """From 2^17 rows on the grid encoding's backward pass orders the batch by cell and scatters over the ordered points. The
    gradient of the table is a sum over rows: the large batch's gradient equals the sum of the gradients of its two halves
    (each below the threshold, scattered in the caller's order) up to fp32 rounding of sums in another order."""
    n = 1 << 17
    cfg = {"otype": "HashGrid", "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 15, "base_resolution": 16, "per_level_scale": 1.5}
    torch.manual_seed(6)
    enc = tcnn.Encoding(2, cfg, dtype=torch.float32)
    with torch.no_grad():
        enc.params.copy_(torch.rand_like(enc.params) * 2 - 1)
    x = torch.rand((n, 2), device=DEVICE)
    w = torch.randn((n, enc.n_output_dims), device=DEVICE)

    def grad_of(rows):
        enc.params.grad = None
        (enc(x[rows]).float() * w[rows]).sum().backward()
        return enc.params.grad.clone()

    whole = grad_of(slice(0, n))
    halves = grad_of(slice(0, n // 2)) + grad_of(slice(n // 2, n))
    scale = float(halves.abs().max())
    assert scale > 1.0
    assert float((whole - halves).abs().max()) <= 2e-5 * scale


def test_nerf_style_directional_network(tcnn):
    """test/python/test_nerf_settings.py:80-86 of the reference: spherical harmonics of degree 4 feeding a network."""
    model = tcnn.NetworkWithInputEncoding(3, 3, net_config(64, 2), {"otype": "SphericalHarmonics", "degree": 4}, dtype=torch.bfloat16)
    x = torch.rand((1000, 3), device=DEVICE)
    y = model(x)
    assert y.shape == (1000, 3) and torch.isfinite(y.float()).all()
    y.float().sum().backward()
    assert model.network.params.grad is not None and torch.isfinite(model.network.params.grad).all()


def test_image_learning_sample(tcnn, monkeypatch):
    """The sample under tiny-dpcpp-nn_amd/samples (counterpart of the reference's mlp_learning_an_image_pytorch.py) learns its
    procedural image: 200 steps bring the mean squared error of the rendered image below 1e-3."""
    import importlib.util
    import os
    import sys

    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tiny-dpcpp-nn_amd", "samples", "mlp_learning_an_image.py")
    spec = importlib.util.spec_from_file_location("mlp_learning_an_image", path)
    sample = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(sample)
    monkeypatch.setattr(sys, "argv", ["mlp_learning_an_image.py", "--n_steps", "200", "--seed", "3"])
    assert sample.main() < 1e-3


def test_image_learning_sample_on_a_picture_file(tcnn, monkeypatch, tmp_path):
    """--image: the sample learns a picture read from a file (the reference's sample learns samples/data/images/albert.jpg,
    samples/mlp_learning_an_image_pytorch.py:128-261; here a small picture written on the spot). The bilinear lookup gives
    the pixel values at pixel positions and their means half-way between."""
    import importlib.util
    import os
    import sys

    from PIL import Image

    h, w = 48, 64
    yy, xx = np.mgrid[0:h, 0:w]
    pic = np.stack([(xx * 255 // (w - 1)), (yy * 255 // (h - 1)), ((xx // 8 + yy // 8) % 2) * 200], axis=2).astype(np.uint8)
    path_png = str(tmp_path / "picture.png")
    Image.fromarray(pic, "RGB").save(path_png)
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tiny-dpcpp-nn_amd", "samples", "mlp_learning_an_image.py")
    spec = importlib.util.spec_from_file_location("mlp_learning_an_image_picture", path)
    sample = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(sample)
    target = sample.PictureTarget(path_png, DEVICE)
    at_pixels = torch.tensor([[5 / w, 7 / h], [0.0, 0.0], [(w - 1) / w, (h - 1) / h], [5.5 / w, 7 / h], [1.0, 1.0]], device=DEVICE)
    got = target(at_pixels).cpu().numpy() * 255
    np.testing.assert_allclose(got[0], pic[7, 5], atol=1e-3)
    np.testing.assert_allclose(got[1], pic[0, 0], atol=1e-3)
    np.testing.assert_allclose(got[2], pic[h - 1, w - 1], atol=1e-3)
    np.testing.assert_allclose(got[3], (pic[7, 5].astype(np.float64) + pic[7, 6]) / 2, atol=1e-3)
    np.testing.assert_allclose(got[4], pic[h - 1, w - 1], atol=1e-3)
    monkeypatch.setattr(sys, "argv", ["mlp_learning_an_image.py", "--n_steps", "300", "--image", path_png, "--seed", "3"])
    assert sample.main() < 3e-3
