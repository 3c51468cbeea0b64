"""numpy-in / numpy-out wrappers around oracle/libtnn_oracle.so: test infrastructure, used by the tests, the smoke check and
the benchmark's parity check and CPU baseline; never by the product."""
import ctypes
from ctypes import c_float, c_int, c_size_t, c_uint32, c_void_p

import numpy as np

BF16, FP16, FP32 = 0, 1, 2
ACT = {"relu": 0, "sigmoid": 4, "none": 8, "linear": 8}
GRID_TYPE = {"Hash": 0, "Dense": 1, "Tiled": 2}
HASH = {"Prime": 0, "CoherentPrime": 1, "ReversedPrime": 2, "Rng": 3}
INTERP = {"Nearest": 0, "Linear": 1, "Smoothstep": 2}


def _p(a):
    return a.ctypes.data_as(c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _f64(a):
    return np.ascontiguousarray(a, dtype=np.float64)


class Oracle:
    def __init__(self, path):
        L = self.L = ctypes.CDLL(path)
        L.tnn_oracle_round.argtypes = [c_void_p, c_void_p, c_size_t, c_int]
        L.tnn_oracle_to_packed_layout_coord.argtypes = [ctypes.c_uint] * 3
        L.tnn_oracle_to_packed_layout_coord.restype = ctypes.c_uint
        L.tnn_oracle_from_packed_layout_coord.argtypes = [ctypes.c_uint] * 3
        L.tnn_oracle_from_packed_layout_coord.restype = ctypes.c_uint
        for n in ("pack_weights", "unpack_weights", "packed_transpose", "pack_and_transpose"):
            getattr(L, "tnn_oracle_" + n).argtypes = [c_void_p, c_void_p, c_int, c_int]
        L.tnn_oracle_zero_weights_padding.argtypes = [c_void_p, c_int, c_int, c_int, c_int, c_int]
        L.tnn_oracle_mlp_forward_f64.argtypes = [c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p]
        L.tnn_oracle_mlp_backward_f64.argtypes = [c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_size_t,
                                                  c_void_p, c_void_p, c_void_p]
        L.tnn_oracle_mlp_forward_T.argtypes = [c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p, c_int]
        L.tnn_oracle_mlp_backward_T.argtypes = [c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_size_t,
                                                c_void_p, c_void_p, c_void_p, c_int]
        L.tnn_oracle_l2_loss.argtypes = [c_int, c_void_p, c_void_p, c_size_t, c_float, c_void_p, c_void_p]
        L.tnn_oracle_adam_step.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_float, c_float, c_float, c_float]
        L.tnn_oracle_grid_offsets.argtypes = [c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p, c_void_p]
        L.tnn_oracle_grid_indices.argtypes = [c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p, c_void_p]
        L.tnn_oracle_grid_forward.argtypes = [c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p, c_void_p,
                                              c_size_t, c_void_p, c_int]
        L.tnn_oracle_grid_backward.argtypes = [c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p, c_void_p,
                                               c_size_t, c_int, c_void_p]
        L.tnn_oracle_identity_forward.argtypes = [c_void_p, c_int, c_float, c_float, c_size_t, c_void_p, c_int]
        L.tnn_oracle_frequency_forward.argtypes = [c_void_p, c_int, c_int, c_size_t, c_void_p, c_int, c_void_p]
        L.tnn_oracle_frequency_backward.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int, c_size_t, c_void_p]
        L.tnn_oracle_sh_explicit16.argtypes = [ctypes.c_double] * 3 + [c_void_p]
        L.tnn_oracle_sh_forward.argtypes = [c_int, c_void_p, c_size_t, c_void_p, c_int]
        L.tnn_oracle_num_threads.restype = c_int
        L.tnn_oracle_set_num_threads.argtypes = [c_int]

    # --- rounding -------------------------------------------------------------------------
    def round(self, a, dtype):
        a = _f32(a)
        out = np.empty_like(a)
        self.L.tnn_oracle_round(_p(a), _p(out), a.size, dtype)
        return out

    def splitmix64(self, seed, index):
        self.L.tnn_oracle_splitmix64.restype = ctypes.c_uint64
        self.L.tnn_oracle_splitmix64.argtypes = [ctypes.c_uint64, ctypes.c_uint64]
        return int(self.L.tnn_oracle_splitmix64(seed, index))

    def fill_uniform(self, n, lo, hi, seed, first_index, dtype):
        out = np.empty(n, np.float32)
        self.L.tnn_oracle_fill_uniform.restype = None
        self.L.tnn_oracle_fill_uniform.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_float, ctypes.c_uint64,
                                                   ctypes.c_uint64, ctypes.c_int]
        self.L.tnn_oracle_fill_uniform(_p(out), n, lo, hi, seed, first_index, dtype)
        return out

    def num_threads(self):
        return self.L.tnn_oracle_num_threads()

    def set_num_threads(self, n):
        self.L.tnn_oracle_set_num_threads(n)

    # --- packing --------------------------------------------------------------------------
    def to_packed(self, idx, rows, cols):
        return self.L.tnn_oracle_to_packed_layout_coord(idx, rows, cols)

    def from_packed(self, idx, rows, cols):
        return self.L.tnn_oracle_from_packed_layout_coord(idx, rows, cols)

    def _perm(self, name, a, n_mats, W):
        a = _f32(a)
        out = np.zeros_like(a)
        getattr(self.L, "tnn_oracle_" + name)(_p(a), _p(out), n_mats, W)
        return out

    def pack_weights(self, unpacked, n_mats, W):
        return self._perm("pack_weights", unpacked, n_mats, W)

    def unpack_weights(self, packed, n_mats, W):
        return self._perm("unpack_weights", packed, n_mats, W)

    def packed_transpose(self, packed, W):
        return self._perm("packed_transpose", packed, W, W)  # (rows, cols)

    def pack_and_transpose(self, raw, W):
        return self._perm("pack_and_transpose", raw, W, W)

    def zero_weights_padding(self, packed, n_mats, W, n_in, n_out, use_bias):
        packed = _f32(packed).copy()
        rc = self.L.tnn_oracle_zero_weights_padding(_p(packed), n_mats, W, n_in, n_out, int(use_bias))
        if rc:
            raise ValueError("zero_weights_padding rejected the widths")
        return packed

    # --- MLP ------------------------------------------------------------------------------
    def mlp_forward_f64(self, W, n_mats, act, out_act, w, x):
        w, x = _f64(w), _f64(x)
        M = x.shape[0]
        out = np.empty((n_mats + 1, M, W), np.float64)
        self.L.tnn_oracle_mlp_forward_f64(W, n_mats, ACT[act], ACT[out_act], _p(w), _p(x), M, _p(out))
        return out

    def mlp_backward_f64(self, W, n_mats, act, out_act, w, layer_outputs, dLdy, want_dx=True):
        w, lo, g = _f64(w), _f64(layer_outputs), _f64(dLdy)
        M = g.shape[0]
        deltas = np.empty((n_mats, M, W), np.float64)
        dW = np.empty((n_mats, W, W), np.float64)
        dX = np.empty((M, W), np.float64) if want_dx else None
        self.L.tnn_oracle_mlp_backward_f64(W, n_mats, ACT[act], ACT[out_act], _p(w), _p(lo), _p(g), M, _p(deltas), _p(dW),
                                           _p(dX) if want_dx else None)
        return deltas, dW, dX

    def mlp_forward_T(self, dtype, W, n_mats, act, out_act, w, x, store_interm=True):
        w, x = _f32(w), _f32(x)
        M = x.shape[0]
        out = np.empty((n_mats + 1, M, W) if store_interm else (M, W), np.float32)
        self.L.tnn_oracle_mlp_forward_T(dtype, W, n_mats, ACT[act], ACT[out_act], _p(w), _p(x), M, _p(out), int(store_interm))
        return out

    def mlp_backward_T(self, dtype, W, n_mats, act, out_act, w, interm_fwd, dLdy, want_dx=True, round_dw=True):
        w, f, g = _f32(w), _f32(interm_fwd), _f32(dLdy)
        M = g.shape[0]
        ib = np.empty((n_mats, M, W), np.float32)
        dW = np.empty((n_mats, W, W), np.float32)
        dX = np.empty((M, W), np.float32) if want_dx else None
        self.L.tnn_oracle_mlp_backward_T(dtype, W, n_mats, ACT[act], ACT[out_act], _p(w), _p(f), _p(g), M, _p(ib), _p(dW),
                                         _p(dX) if want_dx else None, int(round_dw))
        return ib, dW, dX

    def l2_loss(self, dtype, pred, target, loss_scale):
        pred, target = _f32(pred), _f32(target)
        values = np.empty_like(pred)
        grads = np.empty_like(pred)
        self.L.tnn_oracle_l2_loss(dtype, _p(pred), _p(target), pred.size, loss_scale, _p(values), _p(grads))
        return values, grads

    def adam_step(self, param, m, v, grad, step, lr, beta1, beta2, eps):
        param, m, v = _f32(param).copy(), _f32(m).copy(), _f32(v).copy()
        grad = _f32(grad)
        self.L.tnn_oracle_adam_step(_p(param), _p(m), _p(v), _p(grad), param.size, step, lr, beta1, beta2, eps)
        return param, m, v

    # --- grid -----------------------------------------------------------------------------
    def grid_offsets(self, n_dims, n_levels, log2_hashmap_size, base_resolution, per_level_scale, grid_type="Hash"):
        off = np.zeros(n_levels + 1, np.uint32)
        sc = np.zeros(n_levels, np.float32)
        res = np.zeros(n_levels, np.uint32)
        rc = self.L.tnn_oracle_grid_offsets(n_dims, n_levels, log2_hashmap_size, base_resolution, per_level_scale,
                                            GRID_TYPE[grid_type], _p(off), _p(sc), _p(res))
        if rc:
            raise ValueError("grid_offsets")
        return off, sc, res

    def grid_indices(self, cfg, x, want_cells=False):
        x = _f32(x)
        M = x.shape[0]
        D, L = cfg["n_dims"], cfg["n_levels"]
        idx = np.empty((M, L, 1 << D), np.uint32)
        cells = np.empty((M, L, D), np.uint32) if want_cells else None
        rc = self.L.tnn_oracle_grid_indices(D, L, cfg["log2_hashmap_size"], cfg["base_resolution"], cfg["per_level_scale"],
                                            GRID_TYPE[cfg.get("grid_type", "Hash")], HASH[cfg.get("hash", "CoherentPrime")],
                                            INTERP[cfg.get("interpolation", "Linear")], _p(x), M, _p(idx),
                                            _p(cells) if want_cells else None)
        if rc:
            raise ValueError("grid_indices")
        return (idx, cells) if want_cells else idx

    def grid_forward(self, cfg, table, x, padded_width):
        x, table = _f32(x), _f32(table)
        M = x.shape[0]
        out = np.full((M, padded_width), np.nan, np.float32)
        rc = self.L.tnn_oracle_grid_forward(cfg["n_dims"], cfg["n_levels"], cfg["n_features_per_level"], cfg["log2_hashmap_size"],
                                            cfg["base_resolution"], cfg["per_level_scale"], GRID_TYPE[cfg.get("grid_type", "Hash")],
                                            HASH[cfg.get("hash", "CoherentPrime")], INTERP[cfg.get("interpolation", "Linear")],
                                            _p(table), _p(x), M, _p(out), padded_width)
        if rc:
            raise ValueError("grid_forward")
        return out

    def grid_backward(self, cfg, x, dLdy, n_params):
        x, dLdy = _f32(x), _f32(dLdy)
        M = x.shape[0]
        grad = np.full(n_params, np.nan, np.float32)
        rc = self.L.tnn_oracle_grid_backward(cfg["n_dims"], cfg["n_levels"], cfg["n_features_per_level"], cfg["log2_hashmap_size"],
                                             cfg["base_resolution"], cfg["per_level_scale"], GRID_TYPE[cfg.get("grid_type", "Hash")],
                                             HASH[cfg.get("hash", "CoherentPrime")], INTERP[cfg.get("interpolation", "Linear")],
                                             _p(x), _p(dLdy), M, dLdy.shape[1], _p(grad))
        if rc:
            raise ValueError("grid_backward")
        return grad

    # --- encodings without parameters -------------------------------------------------------
    def identity_forward(self, x, scale, offset, padded_width):
        x = _f32(x)
        out = np.empty((x.shape[0], padded_width), np.float32)
        self.L.tnn_oracle_identity_forward(_p(x), x.shape[1], scale, offset, x.shape[0], _p(out), padded_width)
        return out

    def frequency_forward(self, x, n_freq, padded_width, want_dy_dx=False):
        x = _f32(x)
        M, D = x.shape
        out = np.empty((M, padded_width), np.float32)
        dy = np.empty((M, D * n_freq * 2), np.float32) if want_dy_dx else None
        self.L.tnn_oracle_frequency_forward(_p(x), D, n_freq, M, _p(out), padded_width, _p(dy) if want_dy_dx else None)
        return (out, dy) if want_dy_dx else out

    def frequency_backward(self, dLdy, dy_dx, n_dims, n_freq):
        dLdy, dy_dx = _f32(dLdy), _f32(dy_dx)
        M = dLdy.shape[0]
        out = np.empty((M, n_dims), np.float32)
        self.L.tnn_oracle_frequency_backward(_p(dLdy), dLdy.shape[1], _p(dy_dx), n_dims, n_freq, M, _p(out))
        return out

    def sh_explicit16(self, x, y, z):
        out = np.empty(16, np.float64)
        self.L.tnn_oracle_sh_explicit16(float(x), float(y), float(z), _p(out))
        return out

    def sh_forward(self, degree, x, padded_width):
        x = _f32(x)
        out = np.full((x.shape[0], padded_width), np.nan, np.float32)
        if self.L.tnn_oracle_sh_forward(degree, _p(x), x.shape[0], _p(out), padded_width):
            raise ValueError("sh_forward")
        return out
