"""Tensor-level wrappers over the C ABI of libtnn_hip.so (tiny_dpcpp_nn._lib): device buffers come from torch, every
compute call goes through the library. Used by the benchmark, the smoke check and the GPU tests. There is no fallback: a
missing library or GPU raises."""
import ctypes

import numpy as np
import torch

from tiny_dpcpp_nn import _lib

BF16, FP16, FP32 = _lib.TNN_BF16, _lib.TNN_FP16, _lib.TNN_FP32
TORCH_DT = {BF16: torch.bfloat16, FP16: torch.float16, FP32: torch.float32}
ACT = {"relu": _lib.ACT_RELU, "sigmoid": _lib.ACT_SIGMOID, "none": _lib.ACT_NONE}
GRID_TYPE = {"Hash": 0, "Dense": 1, "Tiled": 2}
HASH = {"Prime": 0, "CoherentPrime": 1, "ReversedPrime": 2, "Rng": 3}
INTERP = {"Nearest": 0, "Linear": 1, "Smoothstep": 2}


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


class Harness:
    def __init__(self):
        self.lib = _lib.load()
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible: the HIP path cannot run (and nothing else may stand in for it)")
        self.dev = torch.device("cuda:0")
        _lib.check(self.lib.tnn_device_check())

    # ------------------------------------------------------------------------------
    def stream(self):
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def sync(self):
        torch.cuda.synchronize()

    def dev_tensor(self, a, dtype):
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(self.dev).to(TORCH_DT[dtype]).contiguous()

    def host(self, t):
        return t.detach().to(torch.float32).cpu().numpy()

    def empty(self, shape, dtype, fill=None):
        t = torch.empty(shape, dtype=TORCH_DT[dtype], device=self.dev)
        if fill is not None:
            t.fill_(fill)
        return t

    # ------------------------------------------------------------------------------
    def mlp_desc(self, dtype, W, n_hidden, act, out_act):
        return _lib.MlpDesc(dtype, W, n_hidden, ACT[act] if isinstance(act, str) else act,
                            ACT[out_act] if isinstance(out_act, str) else out_act)

    def pack(self, dtype, W, n_mats, unpacked_t):
        out = torch.empty_like(unpacked_t)
        _lib.check(self.lib.tnn_pack_weights(dtype, W, n_mats, ptr(unpacked_t), ptr(out), self.stream()))
        return out

    def prepare(self, desc, w_unpacked_np):
        """unpacked [n_mats][k][n] weights (numpy) -> (packed, prepared_fwd, prepared_bwd) device tensors"""
        n_mats = desc.n_hidden_layers + 1
        unp = self.dev_tensor(np.asarray(w_unpacked_np).reshape(-1), desc.dtype)
        packed = self.pack(desc.dtype, desc.width, n_mats, unp)
        return (packed,) + self.prepare_packed(desc, packed)

    def prepare_packed(self, desc, packed_t, src_is_fp32=False):
        nbytes = self.lib.tnn_mlp_prepared_bytes(ctypes.byref(desc))
        assert nbytes > 0
        fwd = torch.empty(nbytes // 2, dtype=TORCH_DT[desc.dtype], device=self.dev)
        bwd = torch.empty(nbytes // 2, dtype=TORCH_DT[desc.dtype], device=self.dev)
        _lib.check(self.lib.tnn_mlp_prepare_weights(ctypes.byref(desc), ptr(packed_t), int(src_is_fp32), ptr(fwd), ptr(bwd), self.stream()))
        return fwd, bwd

    def inference(self, desc, prep_fwd, x_t, out=None):
        M = x_t.shape[0]
        y = out if out is not None else torch.empty_like(x_t)
        _lib.check(self.lib.tnn_mlp_inference(ctypes.byref(desc), ptr(prep_fwd), ptr(x_t), ptr(y), M, self.stream()))
        return y

    def forward(self, desc, prep_fwd, x_t):
        M, W = x_t.shape
        interm = torch.full((desc.n_hidden_layers + 2, M, W), float("nan"), dtype=x_t.dtype, device=self.dev)
        _lib.check(self.lib.tnn_mlp_forward(ctypes.byref(desc), ptr(prep_fwd), ptr(x_t), ptr(interm), M, self.stream()))
        return interm

    def backward(self, desc, prep_bwd, dLdy_t, interm_fwd_t, want_interm=True, want_dx=True, dw_fp32=False):
        M, W = dLdy_t.shape
        n_mats = desc.n_hidden_layers + 1
        ws_bytes = self.lib.tnn_mlp_backward_workspace_bytes(ctypes.byref(desc), M)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=self.dev)
        ib = torch.full((n_mats, M, W), float("nan"), dtype=dLdy_t.dtype, device=self.dev) if want_interm else None
        dW = torch.full((n_mats, W, W), float("nan"), dtype=torch.float32 if dw_fp32 else dLdy_t.dtype, device=self.dev)
        dX = torch.full((M, W), float("nan"), dtype=dLdy_t.dtype, device=self.dev) if want_dx else None
        _lib.check(self.lib.tnn_mlp_backward(ctypes.byref(desc), ptr(prep_bwd), ptr(dLdy_t), ptr(interm_fwd_t), ptr(ib), ptr(dW),
                                             int(dw_fp32), ptr(dX), M, ptr(ws), ws_bytes, self.stream()))
        return ib, dW, dX

    def backward_recompute(self, desc, prep_fwd, prep_bwd, x_t, dLdy_t, want_dx=True, dw_fp32=True):
        """Weight gradients (and dL/dx) for a given dL/dy with the forward pass formed again on chip (tnn_mlp_backward_recompute)."""
        M, W = x_t.shape
        n_mats = desc.n_hidden_layers + 1
        ws_bytes = self.lib.tnn_mlp_train_step_workspace_bytes(ctypes.byref(desc), M)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=self.dev)
        dW = torch.full((n_mats, W, W), float("nan"), dtype=torch.float32 if dw_fp32 else x_t.dtype, device=self.dev)
        dX = torch.full((M, W), float("nan"), dtype=x_t.dtype, device=self.dev) if want_dx else None
        _lib.check(self.lib.tnn_mlp_backward_recompute(ctypes.byref(desc), ptr(prep_fwd), ptr(prep_bwd), ptr(x_t), ptr(dLdy_t), ptr(dW), int(dw_fp32),
                                                       ptr(dX), M, ptr(ws), ws_bytes, self.stream()))
        return dW, dX

    def l2_loss(self, dtype, pred_t, targets_t, loss_scale, want_values=True):
        n = pred_t.numel()
        values = torch.empty(pred_t.shape, dtype=torch.float32, device=self.dev) if want_values else None
        grads = torch.empty_like(pred_t)
        _lib.check(self.lib.tnn_l2_loss(dtype, ptr(pred_t), ptr(targets_t), n, loss_scale, ptr(values), ptr(grads), self.stream()))
        return values, grads

    def train_step_l2(self, desc, prep_fwd, prep_bwd, x_t, targets_t, loss_scale, want_y=True, want_dx=True, dw_fp32=True, ws=None):
        M, W = x_t.shape
        n_mats = desc.n_hidden_layers + 1
        ws_bytes = self.lib.tnn_mlp_train_step_workspace_bytes(ctypes.byref(desc), M)
        if ws is None:
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=self.dev)
        y = torch.empty_like(x_t) if want_y else None
        loss = torch.full((1,), float("nan"), dtype=torch.float32, device=self.dev)
        dW = torch.full((n_mats, W, W), float("nan"), dtype=torch.float32 if dw_fp32 else x_t.dtype, device=self.dev)
        dX = torch.empty_like(x_t) if want_dx else None
        _lib.check(self.lib.tnn_mlp_train_step_l2(ctypes.byref(desc), ptr(prep_fwd), ptr(prep_bwd), ptr(x_t), ptr(targets_t), loss_scale,
                                                  ptr(y), ptr(loss), ptr(dW), int(dw_fp32), ptr(dX), M, ptr(ws), ws.numel(), self.stream()))
        return y, loss, dW, dX

    def adam_step(self, param, m, v, grad, grad_dtype, grad_scale, step, lr, b1, b2, eps, param_T=None, param_T_dtype=BF16):
        _lib.check(self.lib.tnn_adam_step(ptr(param), ptr(m), ptr(v), ptr(grad), grad_dtype, grad_scale, param.numel(), step, lr, b1, b2,
                                          eps, ptr(param_T), param_T_dtype, self.stream()))

    # ------------------------------------------------------------------------------
    def grid_desc(self, cfg, param_dtype=FP32):
        d = _lib.GridDesc()
        _lib.check(self.lib.tnn_grid_desc_init(ctypes.byref(d), cfg["n_dims"], cfg["n_levels"], cfg["n_features_per_level"],
                                               cfg["log2_hashmap_size"], cfg["base_resolution"], cfg["per_level_scale"],
                                               GRID_TYPE[cfg.get("grid_type", "Hash")], HASH[cfg.get("hash", "CoherentPrime")],
                                               INTERP[cfg.get("interpolation", "Linear")], param_dtype))
        return d

    def grid_n_params(self, d):
        return self.lib.tnn_grid_n_params(ctypes.byref(d))

    def grid_forward(self, d, x_t, table_t, padded_width, out_dtype=FP32, out=None):
        M = x_t.shape[0]
        if out is None:
            out = torch.full((M, padded_width), float("nan"), dtype=TORCH_DT[out_dtype], device=self.dev)
        _lib.check(self.lib.tnn_grid_forward(ctypes.byref(d), ptr(x_t), ptr(table_t), ptr(out), out_dtype, padded_width, M, self.stream()))
        return out

    def grid_order(self, d, x_t):
        """Cell order of the points: the buffer tnn_grid_forward_ordered reads (records first, then scratch)."""
        M = x_t.shape[0]
        nbytes = self.lib.tnn_grid_order_bytes(ctypes.byref(d), M)
        buf = torch.empty(nbytes, dtype=torch.uint8, device=self.dev)
        _lib.check(self.lib.tnn_grid_order_points(ctypes.byref(d), ptr(x_t), M, ptr(buf), nbytes, self.stream()))
        return buf

    def grid_forward_ordered(self, d, order_t, table_t, padded_width, M, out_dtype=FP32, out=None):
        if out is None:
            out = torch.full((M, padded_width), float("nan"), dtype=TORCH_DT[out_dtype], device=self.dev)
        _lib.check(self.lib.tnn_grid_forward_ordered(ctypes.byref(d), ptr(order_t), ptr(table_t), ptr(out), out_dtype, padded_width, M,
                                                     self.stream()))
        return out

    def grid_mlp_inference(self, gd, desc, x_t, table_t, prep_fwd):
        M = x_t.shape[0]
        y = torch.full((M, desc.width), float("nan"), dtype=TORCH_DT[desc.dtype], device=self.dev)
        _lib.check(self.lib.tnn_grid_mlp_inference(ctypes.byref(gd), ctypes.byref(desc), ptr(x_t), ptr(table_t), ptr(prep_fwd), ptr(y), M,
                                                   self.stream()))
        return y

    def grid_mlp_inference_ordered(self, gd, desc, order_t, table_t, prep_fwd, M):
        y = torch.full((M, desc.width), float("nan"), dtype=TORCH_DT[desc.dtype], device=self.dev)
        _lib.check(self.lib.tnn_grid_mlp_inference_ordered(ctypes.byref(gd), ctypes.byref(desc), ptr(order_t), ptr(table_t), ptr(prep_fwd), ptr(y),
                                                           M, self.stream()))
        return y

    def grid_backward(self, d, x_t, dLdy_t, dy_dtype, grad_t=None, overwrite=True):
        M, pw = dLdy_t.shape
        if grad_t is None:
            grad_t = torch.full((self.grid_n_params(d),), 0.123, dtype=torch.float32, device=self.dev)
        _lib.check(self.lib.tnn_grid_backward(ctypes.byref(d), ptr(x_t), ptr(dLdy_t), dy_dtype, pw, ptr(grad_t), int(overwrite), M, self.stream()))
        return grad_t

    def grid_backward_ordered(self, d, order_t, dLdy_t, dy_dtype, grad_t=None, overwrite=True):
        M, pw = dLdy_t.shape
        if grad_t is None:
            grad_t = torch.full((self.grid_n_params(d),), 0.123, dtype=torch.float32, device=self.dev)
        _lib.check(self.lib.tnn_grid_backward_ordered(ctypes.byref(d), ptr(order_t), ptr(dLdy_t), dy_dtype, pw, ptr(grad_t), int(overwrite), M,
                                                      self.stream()))
        return grad_t

    # ------------------------------------------------------------------------------
    def identity_forward(self, x_t, scale, offset, padded_width, out_dtype=FP32):
        M, D = x_t.shape
        out = torch.full((M, padded_width), float("nan"), dtype=TORCH_DT[out_dtype], device=self.dev)
        _lib.check(self.lib.tnn_identity_forward(ptr(x_t), D, scale, offset, ptr(out), out_dtype, padded_width, M, self.stream()))
        return out

    def frequency_forward(self, x_t, n_freq, padded_width, out_dtype=FP32, want_dy_dx=False):
        M, D = x_t.shape
        out = torch.full((M, padded_width), float("nan"), dtype=TORCH_DT[out_dtype], device=self.dev)
        dy = torch.full((M, D * n_freq * 2), float("nan"), dtype=torch.float32, device=self.dev) if want_dy_dx else None
        _lib.check(self.lib.tnn_frequency_forward(ptr(x_t), D, n_freq, ptr(out), out_dtype, padded_width, ptr(dy), M, self.stream()))
        return (out, dy) if want_dy_dx else out

    def frequency_backward(self, dLdy_t, dy_dtype, dy_dx_t, n_dims, n_freq):
        M, pw = dLdy_t.shape
        out = torch.full((M, n_dims), float("nan"), dtype=torch.float32, device=self.dev)
        _lib.check(self.lib.tnn_frequency_backward(ptr(dLdy_t), dy_dtype, pw, ptr(dy_dx_t), n_dims, n_freq, ptr(out), M, self.stream()))
        return out

    def sh_forward(self, x_t, degree, padded_width, out_dtype=FP32):
        M = x_t.shape[0]
        out = torch.full((M, padded_width), float("nan"), dtype=TORCH_DT[out_dtype], device=self.dev)
        _lib.check(self.lib.tnn_sh_forward(ptr(x_t), degree, ptr(out), out_dtype, padded_width, M, self.stream()))
        return out

    def grid_indices(self, d, x_t):
        M = x_t.shape[0]
        out = torch.empty((M, d.n_levels, 1 << d.n_dims), dtype=torch.int32, device=self.dev)
        _lib.check(self.lib.tnn_grid_indices(ctypes.byref(d), ptr(x_t), ptr(out), M, self.stream()))
        return out.cpu().numpy().view(np.uint32)
