"""torch.nn.Module front end: Network, Encoding, NetworkWithInputEncoding.

Mirrors dpcpp_bindings/tiny_dpcpp_nn/modules.py of the reference: the autograd function (:65-136), the common
Module base with `.params`, `set_params`, `get_params`, `forward` (:139-261), Network (:264-307), Encoding
(:309-354) and NetworkWithInputEncoding (:357-421). Same constructor arguments, attributes, padding rules
(batch to a multiple of 8, network input to the network width with `use_bias` as the fill value) and loss-scale
handling. The device is PyTorch-ROCm's "cuda" device where the reference uses "xpu".

All compute goes through the extension module `tiny_dpcpp_nn_pybind_module` (HIP kernels); importing this file
fails if that module is not built. There is no PyTorch fallback.
"""
import torch

from .tiny_dpcpp_nn_pybind_module import Activation, create_encoding, create_network

MIN_BATCH_SIZE = 8  # the kernels need the batch size to be a multiple of 8

DEFAULT_DEVICE = "cuda"


def free_temporary_memory():
    """Kept for interface compatibility; the workspaces are owned by the modules."""


def unpad_tensor_to_input_dim(padded_tensor, output_dim):
    _, current_width = padded_tensor.shape
    if output_dim > current_width:
        raise ValueError("input_dim must be less than or equal to the current width of the tensor")
    return padded_tensor[:, :output_dim]


def get_dpcpp_activation(name):
    key = name.lower()
    if key == "relu":
        return Activation.ReLU
    if key == "tanh":
        return Activation.Tanh
    if key == "sigmoid":
        return Activation.Sigmoid
    if key in ("linear", "none"):
        return Activation.Linear
    raise NotImplementedError(f"Activation: {name} not defined")


def to_packed_layout_coord(idx, rows, cols):
    i, j = divmod(idx, cols)
    if i % 2 == 0:
        return i * cols + 2 * j
    return (i - 1) * cols + 2 * j + 1


def from_packed_layout_coord(idx, rows, cols):
    i, j = divmod(idx, cols * 2)
    if j % 2 == 0:
        return (i * 2) * cols + j // 2
    return (i * 2 + 1) * cols + (j - 1) // 2


class _module_function(torch.autograd.Function):
    @staticmethod
    def forward(ctx, native_tnn_module, input, params, info, loss_scale):
        batch_size = input.shape[0]
        if info["is_in_eval_mode"]:
            output = native_tnn_module.inference(input)
        else:
            output = native_tnn_module.fwd(input)
        if batch_size > 0:
            output = output.reshape(batch_size, -1)

        ctx.save_for_backward(input, output, params)
        ctx.info = info
        ctx.native_tnn_module = native_tnn_module
        ctx.loss_scale = loss_scale

        if "output_dim" in info:
            return output[..., : info["output_dim"]]  # the columns beyond output_dim are padding
        return output  # encodings

    @staticmethod
    def backward(ctx, doutput):
        input, _, params = ctx.saved_tensors
        loss_scale = ctx.loss_scale

        if "width" in ctx.info and doutput.shape[1] < ctx.info["width"]:
            doutput = torch.nn.functional.pad(doutput, [0, ctx.info["width"] - doutput.shape[1]])  # zeros for the padding columns

        batch_size = input.shape[0]
        # loss scaling: 1 for bf16, where the two passes over the gradient (here and after the kernels) are skipped
        doutput = (doutput if loss_scale == 1.0 else doutput * loss_scale).contiguous()
        with torch.no_grad():
            if "encoding_config" in ctx.info:
                input_grad = None
                if batch_size == 0:
                    grad = torch.zeros_like(params)
                else:
                    # parameters of encodings are not packed; no gradient w.r.t. the input
                    _, grad = ctx.native_tnn_module.bwd_with_encoding_grad(doutput, input, False, False)
            else:
                if batch_size == 0:
                    input_grad, grad = torch.zeros_like(input), torch.zeros_like(params)
                else:
                    # pack the gradient into the parameter layout; dL/dinput only when autograd asks for it (the product
                    # with the first matrix and a batch-sized store otherwise serve nobody)
                    input_grad, grad = ctx.native_tnn_module.bwd_no_encoding_grad(doutput, True, bool(ctx.needs_input_grad[1]))
                    if input_grad is not None:
                        input_grad = input_grad.reshape(batch_size, -1)

        if grad is not None:
            grad = (grad if loss_scale == 1.0 else grad / loss_scale).reshape(params.shape).to(params.dtype)
        if input_grad is not None and loss_scale != 1.0:
            input_grad = input_grad / loss_scale
        # one entry per argument of forward
        return (None, input_grad, grad, None, None)


class Module(torch.nn.Module):
    def __init__(
        self,
        dtype,  # float for encodings, half precision for networks
        device=DEFAULT_DEVICE,
        store_params_as_full_precision=True,
        use_bias=True,
        init_module=True,
    ):
        super().__init__()
        self.device = device
        self.use_bias = use_bias
        self.dtype = dtype
        self.store_params_as_full_precision = store_params_as_full_precision
        self.loss_scale = 128.0 if dtype == torch.float16 else 1.0

        if not init_module:
            return

        self.tnn_module = self.create_module()

        if self.tnn_module.n_params():
            initial_params = self.tnn_module.initial_params()
            params_dtype = torch.float32 if self.store_params_as_full_precision else self.dtype
            # memory owned by PyTorch, independent of the arrays inside the native module
            self.params = torch.nn.Parameter(initial_params.clone().detach().to(params_dtype), requires_grad=True)
        else:
            print("No params initialised, as n_params = 0. This is correct for Encodings (apart from grid encodings).")
            self.params = torch.nn.Parameter(torch.zeros(1, device=self.device), requires_grad=False)

    def set_params(self, params=None):
        """params given: a flat tensor of unpacked [in][out] matrices (networks) or the table (encodings).
        params None: push `self.params`, which already is in the native (packed) layout."""
        if not self.tnn_module.n_params():
            if params is not None:
                raise RuntimeError("Network has no parameters. Cannot set params")
            return

        pushing_own = params is None
        packed = pushing_own and self.name != "encoding"  # encoding parameters are never packed
        if pushing_own:
            params = self.params
        assert isinstance(params, torch.Tensor), "Params is not a torch.Tensor"

        pushed = params.detach()
        if not (pushed.is_cuda and pushed.dtype in (torch.float32, torch.float16, torch.bfloat16) and self.name != "encoding"):
            pushed = pushed.to(self.dtype)  # a network on the GPU converts to its own type itself, in the kernel that copies
        self.tnn_module.set_params(pushed.contiguous(), packed)

        if not pushing_own:
            # keep the Python-side copy equal to what the native module holds (networks: the packed layout). When the
            # module's own `.params` were pushed the two already agree, and the copy back (a whole table for a grid) is skipped.
            self.params.data.copy_(self.get_params().reshape(self.params.shape))

    def get_params(self):
        """The parameters as the native module holds them (networks: packed layout)."""
        return self.tnn_module.get_params()

    def forward(self, x):
        batch_size, input_dim = x.shape
        padded_batch_size = (batch_size + MIN_BATCH_SIZE - 1) // MIN_BATCH_SIZE * MIN_BATCH_SIZE

        padded_tensor = x if batch_size == padded_batch_size else torch.nn.functional.pad(x, [0, 0, 0, padded_batch_size - batch_size])
        padded_tensor = padded_tensor.to(dtype=self.dtype)

        if self.name == "network" and input_dim != self.width:
            # the bias trick: with use_bias the padding columns hold ones (the native module zeroes the weights
            # of the columns beyond the next multiple of 16), otherwise zeros
            padded_tensor = torch.nn.functional.pad(padded_tensor, [0, self.width - input_dim, 0, 0], "constant", float(self.use_bias))

        info = {"is_in_eval_mode": not self.training}
        if hasattr(self, "n_hidden_layers"):
            info.update(
                {
                    "n_hidden_layers": self.n_hidden_layers - 1,
                    "input_dim": self.n_input_dims,
                    "output_dim": self.n_output_dims,
                    "width": self.width,
                }
            )
        if hasattr(self, "encoding_config"):
            info.update({"encoding_config": self.encoding_config})

        self.set_params()
        output = _module_function.apply(self.tnn_module, padded_tensor.contiguous(), self.params, info, self.loss_scale)
        return output[:batch_size, ...]


class Network(Module):
    def __init__(
        self,
        n_input_dims,
        n_output_dims,
        network_config,
        store_params_as_full_precision=True,
        device=DEFAULT_DEVICE,
        dtype=torch.float16,
        use_bias=True,
    ):
        assert dtype in (torch.float16, torch.bfloat16), f"Only torch.float16 or torch.bfloat16 supported, got: {dtype}"
        self.network_config = network_config
        self.width = self.network_config["n_neurons"]
        self.n_input_dims = n_input_dims
        self.n_output_dims = n_output_dims
        self.n_hidden_layers = self.network_config["n_hidden_layers"]
        self.activation = get_dpcpp_activation(self.network_config["activation"])
        self.output_activation = get_dpcpp_activation(self.network_config["output_activation"])
        self.name = "network"
        super().__init__(
            device=device,
            dtype=dtype,
            store_params_as_full_precision=store_params_as_full_precision,
            use_bias=use_bias,
        )

    def create_module(self):
        return create_network(
            self.n_input_dims,
            self.n_output_dims,
            self.n_hidden_layers,
            self.activation,
            self.output_activation,
            self.width,
            str(self.dtype),
            self.use_bias,
        )


class Encoding(Module):
    def __init__(
        self,
        n_input_dims,
        encoding_config,
        n_output_dims=None,  # None: the encoding's own output width
        device=DEFAULT_DEVICE,
        dtype=torch.float,
        store_params_as_full_precision=True,
    ):
        assert dtype == torch.float, "Only torch.float is currently supported for encoding (the grid gradients are float atomics)"
        self.n_input_dims = n_input_dims
        self.encoding_config = encoding_config
        self.padded_output_dims = n_output_dims
        self.encoding_name = self.encoding_config["otype"]
        self.name = "encoding"

        if "n_dims_to_encode" not in self.encoding_config:
            self.encoding_config["n_dims_to_encode"] = self.n_input_dims

        super().__init__(device=device, dtype=dtype, store_params_as_full_precision=store_params_as_full_precision)

        # only known once the native module exists
        self.n_output_dims = self.tnn_module.n_output_dims()

    def create_module(self):
        return create_encoding(self.encoding_name, self.encoding_config, self.padded_output_dims)


class NetworkWithInputEncoding(Module):
    def __init__(
        self,
        n_input_dims,
        n_output_dims,
        network_config,
        encoding_config,
        device=DEFAULT_DEVICE,
        store_params_as_full_precision=True,
        dtype=torch.float16,
        use_bias=True,
    ):
        assert dtype in (torch.float16, torch.bfloat16), (
            f"Only torch.float16 or torch.bfloat16 supported, got: {dtype}."
            " Note, that dtype here only refers to dtype of Network, the Encoding is always float."
        )
        super().__init__(dtype=dtype, init_module=False)

        self.encoding_config = encoding_config
        self.network_config = network_config
        self.width = self.network_config["n_neurons"]
        self.n_input_dims = n_input_dims
        self.n_output_dims = n_output_dims
        self.n_hidden_layers = self.network_config["n_hidden_layers"]
        self.activation = get_dpcpp_activation(self.network_config["activation"])
        self.output_activation = get_dpcpp_activation(self.network_config["output_activation"])
        self.name = "network_with_encoding"

        self.encoding = Encoding(
            n_input_dims,
            encoding_config,
            device=device,
            dtype=torch.float,
            store_params_as_full_precision=store_params_as_full_precision,
            n_output_dims=network_config["n_neurons"],
        )
        assert self.encoding.n_output_dims == network_config["n_neurons"]
        self.network = Network(
            self.encoding.n_output_dims,
            n_output_dims,
            network_config,
            device=device,
            dtype=dtype,
            store_params_as_full_precision=store_params_as_full_precision,
            use_bias=use_bias,
        )
        self.network_with_encoding = torch.nn.Sequential(self.encoding, self.network)

    @property
    def params(self):
        # the network's parameters; the encoding's are reached through `.encoding.params`
        return self.network.params

    def get_params(self):
        raise RuntimeError("Not implemented.")

    def set_params(self, params=None):
        self.network.set_params(params)

    def forward(self, x):
        if (not self.training and not torch.is_grad_enabled() and x.shape[0] > 0
                and self.network.tnn_module.can_fuse_encoding(self.encoding.tnn_module)):
            return self._fused_inference(x)
        return self.network_with_encoding(x)

    def _fused_inference(self, x):
        """Evaluation without autograd on a grid encoding: encoding and network run as one kernel, the encoded matrix is
        never stored. Same values as the two modules in turn (the reference's only route, modules.py:357-421)."""
        batch_size = x.shape[0]
        padded_batch_size = (batch_size + MIN_BATCH_SIZE - 1) // MIN_BATCH_SIZE * MIN_BATCH_SIZE
        padded = x if batch_size == padded_batch_size else torch.nn.functional.pad(x, [0, 0, 0, padded_batch_size - batch_size])
        self.encoding.set_params()
        self.network.set_params()
        output = self.network.tnn_module.inference_with_encoding(self.encoding.tnn_module, padded.to(torch.float32).contiguous())
        return output.reshape(padded_batch_size, -1)[:batch_size, : self.n_output_dims]
