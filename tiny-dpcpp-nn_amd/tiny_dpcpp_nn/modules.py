"""torch.nn.Module front end of the MI355X implementation: Network, Encoding, NetworkWithInputEncoding.

The public surface is the reference's (dpcpp_bindings/tiny_dpcpp_nn/modules.py: autograd function :65-136, Module base
:139-261, Network :264-307, Encoding :309-354, NetworkWithInputEncoding :357-421): the same class names, constructor
arguments and attributes (`params`, `tnn_module`, `n_input_dims`, `n_output_dims`, `width`, `n_hidden_layers`,
`loss_scale`, ...), the same padding rules (batch rows to a multiple of 8; network input columns to the network width,
filled with ones when `use_bias` and zeros otherwise), the same loss scaling (128 for fp16, 1 for bf16) and the same
layout conventions (`params` of a network is the packed layout, `set_params(tensor)` takes unpacked matrices). The device
is PyTorch-ROCm's "cuda" where the reference has "xpu".

As in the reference (modules.py:253), every forward pushes `params` to the native module first, so that any way of
writing them is seen, `params.data[...] = ...` included. The push is one small kernel on the device. A caller that only
ever updates `params` through operations PyTorch's version counter sees (optimizers, copy_(), load_state_dict) can switch
the push off for unchanged parameters with `module.push_params_every_forward = False`.

One difference in behaviour, a saving: a grid encoding and its network run as one kernel, in evaluation and in training.

All compute goes through the extension module `tiny_dpcpp_nn_pybind_module` (HIP kernels); importing this file fails if it
is not built. There is no PyTorch fallback.
"""
import torch
import torch.nn.functional as F

from .tiny_dpcpp_nn_pybind_module import Activation, create_encoding, create_network, set_initial_weight_seed

MIN_BATCH_SIZE = 8  # the kernels take batches that are multiples of 8 rows
DEFAULT_DEVICE = "cuda"

_ACTIVATIONS = {"relu": Activation.ReLU, "tanh": Activation.Tanh, "sigmoid": Activation.Sigmoid, "linear": Activation.Linear,
                "none": Activation.Linear}
_NETWORK_DTYPES = (torch.float16, torch.bfloat16)


def manual_seed(seed):
    """Networks created from now on get reproducible initial weights: seeds counted up from `seed`. Without this call every
    network is seeded from std::random_device, as in the reference (include/network/Network.h:262-263 there), and two runs of a
    program train different networks. No counterpart in the reference."""
    set_initial_weight_seed(int(seed) & (2 ** 64 - 1))


def free_temporary_memory():
    """Nothing to free: every workspace belongs to a module and goes with it. Kept because callers of the reference call it."""


def get_dpcpp_activation(name):
    try:
        return _ACTIVATIONS[name.lower()]
    except KeyError:
        raise NotImplementedError(f"Activation: {name} not defined") from None


def unpad_tensor_to_input_dim(padded_tensor, output_dim):
    if output_dim > padded_tensor.shape[1]:
        raise ValueError("input_dim must be less than or equal to the current width of the tensor")
    return padded_tensor[:, :output_dim]


def to_packed_layout_coord(idx, rows, cols):
    """Flat index of row-major element `idx` of a rows x cols matrix in the packed parameter layout, where the two rows of
    a pair are interleaved element by element."""
    row, col = divmod(idx, cols)
    return (row & ~1) * cols + 2 * col + (row & 1)


def from_packed_layout_coord(idx, rows, cols):
    """Inverse of to_packed_layout_coord."""
    pair, within = divmod(idx, 2 * cols)
    return (2 * pair + (within & 1)) * cols + within // 2


def _rows_padded(n):
    return -(-n // MIN_BATCH_SIZE) * MIN_BATCH_SIZE


def _pad_rows(x, rows):
    return x if x.shape[0] == rows else F.pad(x, [0, 0, 0, rows - x.shape[0]])


class _NativeCall(torch.autograd.Function):
    """One call into the native module, with the gradients the reference's autograd function returns: for a network, dL/dx
    (only if asked for) and the weight gradients in the packed layout; for an encoding, the gradient of its table."""

    @staticmethod
    def forward(ctx, owner, x, params):
        native = owner.tnn_module
        # A network whose shape has the one-kernel backward pass keeps no activations: its training forward is the inference
        # kernel, and the backward pass forms the activations again on chip from the saved input.
        ctx.recompute = bool(owner._is_network and x.shape[0] > 0 and native.can_recompute_backward())
        y = native.fwd(x) if (owner.training and not ctx.recompute) else native.inference(x)
        ctx.owner = owner
        ctx.save_for_backward(x, params)
        return owner._visible_part(y, x.shape[0])

    @staticmethod
    def backward(ctx, dy):
        owner = ctx.owner
        x, params = ctx.saved_tensors
        scale = owner.loss_scale
        full = owner._native_output_columns()
        if full is not None and dy.shape[1] < full:
            dy = F.pad(dy, [0, full - dy.shape[1]])  # nothing flows back through the padding columns
        if scale != 1.0:
            dy = dy * scale  # fp16: keep the deltas clear of the denormal range inside the kernels
        dy = dy.contiguous()
        dx = None
        with torch.no_grad():
            if x.shape[0] == 0:
                dparams = torch.zeros_like(params)
                if owner._is_network:
                    dx = torch.zeros_like(x)
            elif owner._is_network:
                # weight gradients packed into the parameter layout; dL/dx costs a product with the first matrix and a
                # batch-sized store, so it is asked for only when autograd wants it
                if ctx.recompute:
                    dx, dparams = owner.tnn_module.bwd_recompute(dy, x, True, bool(ctx.needs_input_grad[1]))
                else:
                    dx, dparams = owner.tnn_module.bwd_no_encoding_grad(dy, True, bool(ctx.needs_input_grad[1]))
                if dx is not None:
                    dx = dx.reshape(x.shape[0], -1)
            else:
                # a table is not packed, and positions get no gradient
                _, dparams = owner.tnn_module.bwd_with_encoding_grad(dy, x, False, False)
        if dparams is not None:
            if scale != 1.0:
                dparams = dparams / scale
            dparams = dparams.reshape(params.shape).to(params.dtype)
        if dx is not None and scale != 1.0:
            dx = dx / scale
        return None, dx, dparams


class _EncodedNetworkCall(torch.autograd.Function):
    """A grid encoding and its network as one call in both directions: the forward pass is the fused inference kernel (the
    encoded matrix is never stored), the backward pass forms encoding and activations again on chip and returns the weight
    gradients (packed layout) and the gradient of the table. Positions get no gradient, as in the reference
    (dpcpp_bindings/tiny_dpcpp_nn/modules.py:114-128)."""

    @staticmethod
    def forward(ctx, owner, positions, net_params, table):
        # (the native module puts large batches in cell order and keeps the order for the backward pass)
        y = owner.network.tnn_module.inference_with_encoding(owner.encoding.tnn_module, positions, True)
        ctx.owner = owner
        ctx.save_for_backward(positions, net_params, table)
        return y.reshape(positions.shape[0], -1)[:, : owner.n_output_dims]

    @staticmethod
    def backward(ctx, dy):
        owner = ctx.owner
        positions, net_params, table = ctx.saved_tensors
        scale = owner.network.loss_scale
        dy = F.pad(dy, [0, owner.width - dy.shape[1]]) if dy.shape[1] < owner.width else dy
        if scale != 1.0:
            dy = dy * scale
        with torch.no_grad():
            # positions is a tensor autograd saved: it raises if the tensor was written to since the forward pass, so the cell
            # order formed there (if it was the native module's last) still is the order of these contents
            dnet, dtable = owner.network.tnn_module.bwd_with_encoding(owner.encoding.tnn_module, positions, dy.contiguous(), True, True)
            if scale != 1.0:
                dnet = dnet / scale
                dtable = dtable / scale
        return None, None, dnet.reshape(net_params.shape).to(net_params.dtype), dtable.reshape(table.shape).to(table.dtype)


class Module(torch.nn.Module):
    """Base of the three front-end classes: owns the native module (`tnn_module`) and the PyTorch-side parameter tensor
    `params` (fp32 when `store_params_as_full_precision`, else the module's dtype; a network's is in the packed layout)."""

    _is_network = False

    def __init__(self, dtype, device=DEFAULT_DEVICE, store_params_as_full_precision=True, use_bias=True, init_module=True):
        super().__init__()
        self.dtype = dtype
        self.device = device
        self.use_bias = use_bias
        self.store_params_as_full_precision = store_params_as_full_precision
        self.loss_scale = 128.0 if dtype == torch.float16 else 1.0
        # True (the reference's behaviour): every forward pushes `params` first. False: only when the tensor's identity, storage
        # address or version counter changed since the last push -- a write through `.data` changes none of them and then
        # needs an explicit set_params().
        self.push_params_every_forward = True
        self._pushed = None  # (tensor identity, storage address, version) of `params` when the native module last took it
        if not init_module:
            return
        self.tnn_module = self.create_module()
        if self.tnn_module.n_params() == 0:
            print("No params initialised, as n_params = 0. This is correct for Encodings (apart from grid encodings).")
            self.params = torch.nn.Parameter(torch.zeros(1, device=self.device), requires_grad=False)
            return
        held = torch.float32 if store_params_as_full_precision else dtype
        # PyTorch's own memory, not a view of the native module's arrays
        self.params = torch.nn.Parameter(self.tnn_module.initial_params().detach().clone().to(held), requires_grad=True)

    # ---- what the autograd function asks of its owner ------------------------------------------------------------
    def _visible_output_columns(self):
        return None

    def _visible_part(self, y, rows):
        """The native module's result as [rows, visible columns]; no view is made when it already is that (a slice that keeps
        everything still costs autograd a batch-sized zero fill and a copy on the way back)."""
        if rows > 0 and y.dim() != 2:
            y = y.reshape(rows, -1)
        visible = self._visible_output_columns()
        return y if (visible is None or visible == y.shape[-1]) else y[..., :visible]  # the rest of a network's output row is padding

    def _native_output_columns(self):
        return None

    # ---- parameters ----------------------------------------------------------------------------------------------
    def _params_state(self):
        p = self.params
        return (id(p), p.data_ptr(), p._version)

    def _push(self, tensor, packed):
        t = tensor.detach()
        # a network on the GPU converts fp32 / fp16 / bf16 to its own type in the kernel that copies; everything else is cast here
        if not (self._is_network and t.is_cuda and t.dtype in (torch.float32,) + _NETWORK_DTYPES):
            t = t.to(self.dtype)
        self.tnn_module.set_params(t.contiguous(), packed)

    def set_params(self, params=None):
        """`params` given: a flat tensor of unpacked [in][out] matrices (network) or the table (encoding); it is pushed to the
        native module and `self.params` takes what the module then holds. `None`: push `self.params` as it is (a network's is
        already packed)."""
        if self.tnn_module.n_params() == 0:
            if params is not None:
                raise RuntimeError("Network has no parameters. Cannot set params")
            return
        if params is None:
            self._push(self.params, packed=self._is_network)
        else:
            assert isinstance(params, torch.Tensor), "Params is not a torch.Tensor"
            self._push(params, packed=False)
            with torch.no_grad():
                self.params.copy_(self.get_params().reshape(self.params.shape))
        self._pushed = self._params_state()

    def _push_before_forward(self):
        """What the reference does in front of every forward (modules.py:253): set_params(). With push_params_every_forward
        switched off, only when `params` is known to have changed: in-place updates (optimizer steps, copy_, load_state_dict)
        raise the tensor's version and a replaced tensor has another identity or address; writes through `.data` do neither."""
        if self.tnn_module.n_params() and (self.push_params_every_forward or self._pushed != self._params_state()):
            self.set_params()

    def get_params(self):
        """The parameters as the native module holds them (a network's: packed layout)."""
        return self.tnn_module.get_params()

    # ---- evaluation ----------------------------------------------------------------------------------------------
    def _prepare_input(self, x):
        return _pad_rows(x, _rows_padded(x.shape[0])).to(dtype=self.dtype)

    def forward(self, x):
        batch = x.shape[0]
        self._push_before_forward()
        xin = self._prepare_input(x).contiguous()
        if torch.is_grad_enabled():
            y = _NativeCall.apply(self, xin, self.params)
        else:  # nothing to record: straight to the kernel
            y = self._visible_part(self.tnn_module.inference(xin), xin.shape[0])
        return y if xin.shape[0] == batch else y[:batch]


class Network(Module):
    _is_network = True
    name = "network"

    def __init__(self, n_input_dims, n_output_dims, network_config, store_params_as_full_precision=True, device=DEFAULT_DEVICE,
                 dtype=torch.float16, use_bias=True):
        assert dtype in _NETWORK_DTYPES, f"Only torch.float16 or torch.bfloat16 supported, got: {dtype}"
        self.n_input_dims = n_input_dims
        self.n_output_dims = n_output_dims
        self.network_config = network_config
        self.width = network_config["n_neurons"]
        self.n_hidden_layers = network_config["n_hidden_layers"]
        self.activation = get_dpcpp_activation(network_config["activation"])
        self.output_activation = get_dpcpp_activation(network_config["output_activation"])
        super().__init__(dtype=dtype, device=device, store_params_as_full_precision=store_params_as_full_precision, use_bias=use_bias)

    def create_module(self):
        return create_network(self.n_input_dims, self.n_output_dims, self.n_hidden_layers, self.activation, self.output_activation,
                              self.width, str(self.dtype), self.use_bias)

    def _visible_output_columns(self):
        return self.n_output_dims

    def _native_output_columns(self):
        return self.width

    def _prepare_input(self, x):
        x = super()._prepare_input(x)
        missing = self.width - x.shape[1]
        if missing:
            # the bias trick: ones in the padding columns when use_bias (the native module zeroes the weights of the columns
            # beyond the next multiple of 16), zeros otherwise
            x = F.pad(x, [0, missing], "constant", float(self.use_bias))
        return x


class Encoding(Module):
    name = "encoding"

    def __init__(self, n_input_dims, encoding_config, n_output_dims=None, device=DEFAULT_DEVICE, dtype=torch.float,
                 store_params_as_full_precision=True):
        assert dtype == torch.float, "Only torch.float is currently supported for encoding (the grid gradients are float atomics)"
        self.n_input_dims = n_input_dims
        self.encoding_config = encoding_config
        self.encoding_config.setdefault("n_dims_to_encode", n_input_dims)
        self.encoding_name = encoding_config["otype"]
        self.padded_output_dims = n_output_dims  # None: the encoding's own width
        super().__init__(dtype=dtype, device=device, store_params_as_full_precision=store_params_as_full_precision)
        self.n_output_dims = self.tnn_module.n_output_dims()  # known once the native module exists

    def create_module(self):
        return create_encoding(self.encoding_name, self.encoding_config, self.padded_output_dims)


class NetworkWithInputEncoding(Module):
    name = "network_with_encoding"

    def __init__(self, n_input_dims, n_output_dims, network_config, encoding_config, device=DEFAULT_DEVICE,
                 store_params_as_full_precision=True, dtype=torch.float16, use_bias=True):
        assert dtype in _NETWORK_DTYPES, (f"Only torch.float16 or torch.bfloat16 supported, got: {dtype}."
                                          " Note, that dtype here only refers to dtype of Network, the Encoding is always float.")
        super().__init__(dtype=dtype, init_module=False)
        self.n_input_dims = n_input_dims
        self.n_output_dims = n_output_dims
        self.network_config = network_config
        self.encoding_config = encoding_config
        self.width = network_config["n_neurons"]
        self.n_hidden_layers = network_config["n_hidden_layers"]
        self.activation = get_dpcpp_activation(network_config["activation"])
        self.output_activation = get_dpcpp_activation(network_config["output_activation"])
        # the encoding pads its rows to the network width itself, so the network never pads its input
        self.encoding = Encoding(n_input_dims, encoding_config, n_output_dims=self.width, device=device, dtype=torch.float,
                                 store_params_as_full_precision=store_params_as_full_precision)
        assert self.encoding.n_output_dims == self.width
        self.network = Network(self.width, n_output_dims, network_config, store_params_as_full_precision=store_params_as_full_precision,
                               device=device, dtype=dtype, use_bias=use_bias)
        self.network_with_encoding = torch.nn.Sequential(self.encoding, self.network)

    @property
    def params(self):
        return self.network.params  # the table is `self.encoding.params`

    def get_params(self):
        raise RuntimeError("Not implemented.")

    def set_params(self, params=None):
        self.network.set_params(params)

    def forward(self, x):
        if x.shape[0] == 0:
            return self.network_with_encoding(x)
        net, enc = self.network.tnn_module, self.encoding.tnn_module
        if not torch.is_grad_enabled():
            return self._fused_inference(x) if net.can_fuse_encoding(enc) else self.network_with_encoding(x)
        if net.can_train_with_encoding(enc):
            return self._fused_call(x)
        return self.network_with_encoding(x)

    def _fused_call(self, x):
        """With autograd: one kernel forward (values as the two modules in turn), one kernel plus the scatter backward."""
        batch = x.shape[0]
        rows = _rows_padded(batch)
        self.encoding._push_before_forward()
        self.network._push_before_forward()
        positions = _pad_rows(x.detach(), rows).to(torch.float32).contiguous()
        return _EncodedNetworkCall.apply(self, positions, self.network.params, self.encoding.params)[:batch]

    def _fused_inference(self, x):
        """Without autograd on a grid encoding: one kernel, the encoded matrix is never stored; the values are those of the two
        modules in turn (the reference's only route)."""
        batch = x.shape[0]
        rows = _rows_padded(batch)
        self.encoding._push_before_forward()
        self.network._push_before_forward()
        positions = _pad_rows(x, rows).to(torch.float32).contiguous()
        y = self.network.tnn_module.inference_with_encoding(self.encoding.tnn_module, positions)
        return y.reshape(rows, -1)[:batch, : self.n_output_dims]
