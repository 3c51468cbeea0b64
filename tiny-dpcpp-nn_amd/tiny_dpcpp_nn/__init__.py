"""MI355X-native drop-in for the `tiny_dpcpp_nn` Python package of intel/tiny-dpcpp-nn."""
