"""The tests' handle on the C ABI: the tensor-level wrappers live in the package (tiny_dpcpp_nn.cabi)."""
from tiny_dpcpp_nn.cabi import *  # noqa: F401,F403
from tiny_dpcpp_nn.cabi import Harness, ptr  # noqa: F401
