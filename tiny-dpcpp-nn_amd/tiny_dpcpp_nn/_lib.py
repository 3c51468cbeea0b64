"""ctypes binding of libtnn_hip.so (the C ABI declared in include/tnn_hip.h).

The library is the only compute path: if it is missing, loading raises and nothing falls back to
PyTorch or the CPU.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_size_t, c_uint32, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libtnn_hip.so")

TNN_OK = 0
TNN_ERR_INVALID_ARGUMENT = -1
TNN_ERR_UNSUPPORTED = -2
TNN_ERR_HIP = -3
TNN_ERR_WORKSPACE = -4

TNN_BF16, TNN_FP16, TNN_FP32 = 0, 1, 2

# ordinals of the reference's `enum class Activation` (include/common/common.h:28-38)
ACT_RELU, ACT_LEAKY_RELU, ACT_EXPONENTIAL, ACT_SINE, ACT_SIGMOID, ACT_SQUAREPLUS, ACT_SOFTPLUS, ACT_TANH, ACT_NONE = range(9)

GRID_HASH, GRID_DENSE, GRID_TILED = 0, 1, 2
HASH_PRIME, HASH_COHERENT_PRIME, HASH_REVERSED_PRIME, HASH_RNG = 0, 1, 2, 3
INTERP_NEAREST, INTERP_LINEAR, INTERP_SMOOTHSTEP = 0, 1, 2

TNN_GRID_MAX_LEVELS = 128


class MlpDesc(ctypes.Structure):
    _fields_ = [
        ("dtype", c_int32),
        ("width", c_int32),
        ("n_hidden_layers", c_int32),
        ("activation", c_int32),
        ("output_activation", c_int32),
    ]


class GridDesc(ctypes.Structure):
    _fields_ = [
        ("n_dims", c_uint32),
        ("n_levels", c_uint32),
        ("n_features_per_level", c_uint32),
        ("log2_hashmap_size", c_uint32),
        ("base_resolution", c_uint32),
        ("per_level_scale", c_float),
        ("grid_type", c_uint32),
        ("hash_type", c_uint32),
        ("interpolation", c_uint32),
        ("param_dtype", c_uint32),
        ("offsets", c_uint32 * (TNN_GRID_MAX_LEVELS + 1)),
        ("scales", c_float * TNN_GRID_MAX_LEVELS),
        ("resolutions", c_uint32 * TNN_GRID_MAX_LEVELS),
    ]


# name -> (restype, argtypes); every symbol include/tnn_hip.h declares
SIGNATURES = {
    "tnn_last_error": (c_char_p, []),
    "tnn_abi_version": (c_int, []),
    "tnn_device_check": (c_int, []),
    "tnn_fill": (c_int, [c_int, c_void_p, c_size_t, c_float, c_void_p]),
    "tnn_fill_uniform": (c_int, [c_int, c_void_p, c_size_t, c_float, c_float, ctypes.c_uint64, ctypes.c_uint64, c_void_p]),
    "tnn_cast": (c_int, [c_int, c_void_p, c_int, c_void_p, c_size_t, c_void_p]),
    "tnn_pack_weights": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "tnn_unpack_weights": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "tnn_packed_transpose": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "tnn_pack_and_transpose": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "tnn_zero_weights_padding": (c_int, [POINTER(MlpDesc), c_void_p, c_int, c_int, c_int, c_void_p]),
    "tnn_mlp_prepared_bytes": (c_size_t, [POINTER(MlpDesc)]),
    "tnn_mlp_prepare_weights": (c_int, [POINTER(MlpDesc), c_void_p, c_int, c_void_p, c_void_p, c_void_p]),
    "tnn_mlp_inference": (c_int, [POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "tnn_mlp_forward": (c_int, [POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "tnn_mlp_backward_workspace_bytes": (c_size_t, [POINTER(MlpDesc), c_size_t]),
    "tnn_mlp_backward": (
        c_int,
        [POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p],
    ),
    "tnn_l2_loss": (c_int, [c_int, c_void_p, c_void_p, c_size_t, c_float, c_void_p, c_void_p, c_void_p]),
    "tnn_mlp_train_step_workspace_bytes": (c_size_t, [POINTER(MlpDesc), c_size_t]),
    "tnn_mlp_train_step_l2": (
        c_int,
        [POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
         c_size_t, c_void_p, c_size_t, c_void_p],
    ),
    "tnn_mlp_backward_recompute_supported": (c_int, [ctypes.POINTER(MlpDesc)]),
    "tnn_mlp_backward_recompute": (c_int, [ctypes.POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_size_t,
                                           c_void_p, c_size_t, c_void_p]),
    "tnn_grid_mlp_backward": (c_int, [ctypes.POINTER(GridDesc), ctypes.POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_int, c_void_p, c_int, c_size_t, c_void_p, c_size_t, c_void_p]),
    "tnn_mlp_set_packed_weights": (c_int, [ctypes.POINTER(MlpDesc), c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "tnn_probe_line_gather": (c_int, [c_void_p, c_size_t, c_size_t, c_int, ctypes.c_uint32, c_void_p, c_void_p]),
    "tnn_debug_set_meeting_spin_limit": (c_int, [c_int, ctypes.POINTER(c_int)]),
    "tnn_mlp_train_step_l2_static_max_bytes": (c_size_t, []),
    "tnn_mlp_train_step_l2_static": (
        c_int,
        [POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
         c_size_t, c_void_p],
    ),
    "tnn_adam_step": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_float, c_size_t, c_int, c_float, c_float, c_float, c_float, c_void_p,
         c_int, c_void_p],
    ),
    "tnn_mlp_adam_update": (
        c_int,
        [POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int, c_float, c_float, c_float, c_float, c_void_p,
         c_void_p, c_void_p, c_void_p],
    ),
    "tnn_mlp_train_step_l2_adam": (
        c_int,
        [POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
         c_float, c_float, c_float, c_float, c_void_p, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p, c_void_p],
    ),
    "tnn_grid_desc_init": (
        c_int,
        [POINTER(GridDesc), c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_float, c_uint32, c_uint32, c_uint32, c_uint32],
    ),
    "tnn_grid_n_params": (c_size_t, [POINTER(GridDesc)]),
    "tnn_grid_forward": (c_int, [POINTER(GridDesc), c_void_p, c_void_p, c_void_p, c_int, c_uint32, c_size_t, c_void_p]),
    "tnn_grid_order_bytes": (c_size_t, [POINTER(GridDesc), c_size_t]),
    "tnn_grid_order_points": (c_int, [POINTER(GridDesc), c_void_p, c_size_t, c_void_p, c_size_t, c_void_p]),
    "tnn_grid_forward_ordered": (c_int, [POINTER(GridDesc), c_void_p, c_void_p, c_void_p, c_int, c_uint32, c_size_t, c_void_p]),
    "tnn_grid_backward": (c_int, [POINTER(GridDesc), c_void_p, c_void_p, c_int, c_uint32, c_void_p, c_int, c_size_t, c_void_p]),
    "tnn_grid_backward_ordered": (c_int, [POINTER(GridDesc), c_void_p, c_void_p, c_int, c_uint32, c_void_p, c_int, c_size_t, c_void_p]),
    "tnn_grid_backward_packed": (c_int, [POINTER(GridDesc), c_void_p, c_void_p, c_int, c_uint32, c_void_p, c_int, c_size_t, c_void_p]),
    "tnn_grid_indices": (c_int, [POINTER(GridDesc), c_void_p, c_void_p, c_size_t, c_void_p]),
    "tnn_grid_mlp_inference": (c_int, [POINTER(GridDesc), POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "tnn_grid_mlp_inference_ordered": (c_int, [POINTER(GridDesc), POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "tnn_grid_mlp_supported": (c_int, [POINTER(GridDesc), POINTER(MlpDesc)]),
    "tnn_grid_mlp_train_supported": (c_int, [POINTER(GridDesc), POINTER(MlpDesc)]),
    "tnn_grid_mlp_train_step_workspace_bytes": (c_size_t, [POINTER(GridDesc), POINTER(MlpDesc), c_size_t]),
    "tnn_grid_mlp_train_step_l2_adam": (
        c_int,
        [POINTER(GridDesc), POINTER(MlpDesc), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p,
         c_void_p, c_void_p, c_void_p, c_int, c_float, c_float, c_float, c_float, c_void_p, c_void_p, c_int, c_size_t, c_void_p, c_size_t,
         c_void_p],
    ),
    "tnn_identity_forward": (c_int, [c_void_p, c_uint32, c_float, c_float, c_void_p, c_int, c_uint32, c_size_t, c_void_p]),
    "tnn_frequency_forward": (c_int, [c_void_p, c_uint32, c_uint32, c_void_p, c_int, c_uint32, c_void_p, c_size_t, c_void_p]),
    "tnn_frequency_backward": (c_int, [c_void_p, c_int, c_uint32, c_void_p, c_uint32, c_uint32, c_void_p, c_size_t, c_void_p]),
    "tnn_sh_forward": (c_int, [c_void_p, c_uint32, c_void_p, c_int, c_uint32, c_size_t, c_void_p]),
}


class TnnError(RuntimeError):
    """A C-ABI call returned a negative status. `.status` holds it."""

    def __init__(self, status, message):
        super().__init__(message)
        self.status = status


class TnnInvalidArgument(TnnError, ValueError):
    pass


_lib = None


def load():
    """Loads libtnn_hip.so once and declares every prototype. Raises if the library is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C tiny-dpcpp-nn_amd/csrc` (there is no fallback path)"
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status):
    """Raises for a negative status, with the library's message."""
    if status >= 0:
        return status
    msg = load().tnn_last_error()
    msg = msg.decode() if msg else "tnn error"
    if status == TNN_ERR_INVALID_ARGUMENT:
        raise TnnInvalidArgument(status, msg)
    raise TnnError(status, msg)
