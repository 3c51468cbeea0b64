"""MI355X-native drop-in for the `tiny_dpcpp_nn` Python package of intel/tiny-dpcpp-nn.

Public names are those of the reference (dpcpp_bindings/tiny_dpcpp_nn/__init__.py:1-8), plus `manual_seed` (reproducible initial
weights; the reference seeds every network from std::random_device). They are resolved on first
use, so that `tiny_dpcpp_nn._lib` (the ctypes binding of the C ABI) can be imported without PyTorch.
"""

__all__ = ["free_temporary_memory", "NetworkWithInputEncoding", "Network", "Encoding", "manual_seed"]


def __getattr__(name):
    if name in __all__:
        from . import modules

        return getattr(modules, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
