#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

Default workload (BASELINE config 2, the one the metric is quoted on): one training step of the
width-64, 4-hidden-layer bf16 fused MLP at batch 2^18 -- forward, L2 loss against U[0,1) targets,
backward with weight gradients, Adam (lr 1e-3, betas 0.9/0.99, eps 1e-15) on fp32 master weights and
re-staging of the updated weights for the next step: one tnn_mlp_train_step_l2_adam call, two kernel
launches. Inputs are resident in HBM before the timed region. Prints ONE JSON line.

Other workloads (reported as extra lines only when asked for with --workload):
  infer  BASELINE config 1 shape at batch 2^18: fused inference
  grid   BASELINE config 5 encoding: 3-D hash grid forward, 2^21 points
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tiny-dpcpp-nn_amd"))
sys.path.insert(0, os.path.join(ROOT, "oracle"))  # the checker (cpu_baseline leg and the parity check only)

PEAK_MFMA_BF16 = 2500.0  # TFLOP/s, dense
PEAK_HBM = 8000.0  # GB/s

# HBM-side bytes per launch of each workload's dominant kernel at the default batch sizes, from rocprofv3 counter runs over this
# file (FETCH_SIZE and WRITE_SIZE, one run each, scaled by what the same counter reads for the --copy-calibration kernel:
# x2.000 and x1.000). The summaries with the commands are profiles/mlp_train_fused_kernel.*.txt, profiles/mlp_forward_kernel.*.txt,
# profiles/grid_forward_kernel.*.txt, profiles/grid_mlp_inference_kernel.*.txt and profiles/grid_backward_kernel.*.txt. Not measured live: counters need the profiler.
MEASURED_TRAFFIC_BYTES = {
    ("train", 18): (56937.8 * 2.0 + 20488.0) * 1024,
    ("infer", 18): (16575.2 * 2.0 + 32768.0) * 1024,
    ("train_fb", 18): (98600.2 * 2.0 + 217143.4) * 1024,  # the backward kernel
    ("grid", 21): (6211700.1 * 2.0 + 262135.3) * 1024,
    ("grid_mlp", 21): (6637904.7 * 2.0 + 263960.6) * 1024,
    ("grid_train", 18): (211580.8 * 2.0 + 236762.7) * 1024,  # the scatter kernel; an atomic request counts as a 32-byte write
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # a step takes 15-60 us: the first few hundred run while the clocks still ramp up (58.9 us per training step over 200 steps
    # after 20, 54.0 over 1000 after 200, 53.6 over 2000 after 500), so the defaults time a second of steady state at most
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default="train", choices=["train", "train_fb", "infer", "grid", "grid_mlp", "grid_train"])
    ap.add_argument("--batch-log2", type=int, default=None)
    ap.add_argument("--packed-scatter", action="store_true",
                    help="grid_train only: gradient table in fp16 with one packed atomic per feature pair (tnn_grid_backward_packed)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain copy kernel (tnn_cast fp32 -> fp32, 256 MiB read + 256 MiB written per launch) so that "
                         "hardware byte counters collected over this run can be scaled by what they read for a known transfer")
    return ap.parse_args()


def cpu_baseline_train(oracle, W, n_mats, budget_s=12.0):
    """The oracle's training step (rounding-point restatement) timed on the host cores on a bounded sample."""
    import numpy as np
    from tolerances import BF16

    rng = np.random.default_rng(0)
    lim = np.sqrt(6.0 / (2 * W))
    w = oracle.round(rng.uniform(-lim, lim, (n_mats, W, W)), BF16)
    cores = oracle.num_threads()
    M = 1 << 14
    x = oracle.round(rng.uniform(-1, 1, (M, W)), BF16)
    tg = rng.uniform(0, 1, (M, W)).astype(np.float32)

    def step():
        interm = oracle.mlp_forward_T(BF16, W, n_mats, "relu", "none", w, x)
        _, g = oracle.l2_loss(BF16, interm[-1], tg, 1.0)
        oracle.mlp_backward_T(BF16, W, n_mats, "relu", "none", w, interm, g, want_dx=False, round_dw=False)

    step()
    t0 = time.perf_counter()
    n = 0
    while time.perf_counter() - t0 < budget_s:
        step()
        n += 1
    dt = time.perf_counter() - t0
    return {"value": M * n / dt, "unit": "samples/s", "cores": cores, "kind": "port",
            "sample": f"{n} training steps (forward, L2, backward with dW) of {M} rows each, w64 / 4 hidden layers, bf16 rounding points, OpenMP over rows"}


def cpu_baseline_infer(oracle, W, n_mats, budget_s=12.0):
    import numpy as np
    from tolerances import BF16

    rng = np.random.default_rng(0)
    lim = np.sqrt(6.0 / (2 * W))
    w = oracle.round(rng.uniform(-lim, lim, (n_mats, W, W)), BF16)
    M = 1 << 15
    x = oracle.round(rng.uniform(-1, 1, (M, W)), BF16)
    oracle.mlp_forward_T(BF16, W, n_mats, "relu", "none", w, x, store_interm=False)
    t0 = time.perf_counter()
    n = 0
    while time.perf_counter() - t0 < budget_s:
        oracle.mlp_forward_T(BF16, W, n_mats, "relu", "none", w, x, store_interm=False)
        n += 1
    dt = time.perf_counter() - t0
    return {"value": M * n / dt, "unit": "samples/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{n} inference passes of {M} rows, w64 / 4 hidden layers, bf16 rounding points, OpenMP over rows"}


def cpu_baseline_grid(oracle, cfg, budget_s=12.0):
    import numpy as np
    from tolerances import FP16

    rng = np.random.default_rng(0)
    off, _, _ = oracle.grid_offsets(cfg["n_dims"], cfg["n_levels"], cfg["log2_hashmap_size"], cfg["base_resolution"], cfg["per_level_scale"])
    n = int(off[-1]) * cfg["n_features_per_level"]
    table = oracle.round(rng.uniform(-1e-4, 1e-4, n), FP16)
    M = 1 << 16
    x = rng.uniform(0, 1, (M, cfg["n_dims"])).astype(np.float32)
    oracle.grid_forward(cfg, table, x, 32)
    t0 = time.perf_counter()
    k = 0
    while time.perf_counter() - t0 < budget_s:
        oracle.grid_forward(cfg, table, x, 32)
        k += 1
    dt = time.perf_counter() - t0
    return {"value": M * k / dt, "unit": "points/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{k} forward passes of {M} points through the full 162 MiB table, OpenMP over points"}


def cpu_baseline_grid_mlp(oracle, cfg, w, budget_s=12.0):
    import numpy as np
    from tolerances import FP16

    rng = np.random.default_rng(0)
    off, _, _ = oracle.grid_offsets(cfg["n_dims"], cfg["n_levels"], cfg["log2_hashmap_size"], cfg["base_resolution"], cfg["per_level_scale"])
    n = int(off[-1]) * cfg["n_features_per_level"]
    table = oracle.round(rng.uniform(-1e-4, 1e-4, n), FP16)
    M = 1 << 16
    x = rng.uniform(0, 1, (M, cfg["n_dims"])).astype(np.float32)
    n_mats = w.shape[0]

    def chain():
        enc = oracle.round(oracle.grid_forward(cfg, table, x, 64), FP16)
        return oracle.mlp_forward_T(FP16, 64, n_mats, "relu", "none", w, enc, store_interm=False)

    chain()
    t0 = time.perf_counter()
    k = 0
    while time.perf_counter() - t0 < budget_s:
        chain()
        k += 1
    dt = time.perf_counter() - t0
    return {"value": M * k / dt, "unit": "points/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{k} passes of {M} points: encoding through the full 162 MiB table, then the 4-matrix network, OpenMP over points"}


def cpu_baseline_grid_train(oracle, cfg, w, budget_s=12.0):
    """Config 4's step on the host: encoding, network forward, L2 loss, network backward with dL/d(encoding), scatter into the
    gradient table. (The two Adam updates are elementwise and left out.)"""
    import numpy as np
    from tolerances import FP16

    rng = np.random.default_rng(0)
    off, _, _ = oracle.grid_offsets(cfg["n_dims"], cfg["n_levels"], cfg["log2_hashmap_size"], cfg["base_resolution"], cfg["per_level_scale"])
    n = int(off[-1]) * cfg["n_features_per_level"]
    table = oracle.round(rng.uniform(-1e-4, 1e-4, n), FP16)
    M = 1 << 14
    x = rng.uniform(0, 1, (M, cfg["n_dims"])).astype(np.float32)
    targets = np.zeros((M, 64), np.float32)
    targets[:, :3] = rng.uniform(0, 1, (M, 3))
    n_mats = w.shape[0]

    def step():
        enc = oracle.round(oracle.grid_forward(cfg, table, x, 64), FP16)
        interm = oracle.mlp_forward_T(FP16, 64, n_mats, "relu", "none", w, enc)
        _, grads = oracle.l2_loss(FP16, interm[-1], targets, 128.0)
        _, _, d_enc = oracle.mlp_backward_T(FP16, 64, n_mats, "relu", "none", w, interm, grads, round_dw=False)
        oracle.grid_backward(cfg, x, d_enc, n)

    step()
    t0 = time.perf_counter()
    k = 0
    while time.perf_counter() - t0 < budget_s:
        step()
        k += 1
    dt = time.perf_counter() - t0
    return {"value": M * k / dt, "unit": "samples/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{k} steps of {M} points: encoding, network forward, L2, network backward, scatter into the 7.7 M-entry gradient "
                      "table; OpenMP over points"}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path. Every batch row is independent, so G GPUs would each take "
              "M/G rows with a full copy of the weights and exchange the weight gradients once per step; that is not built. "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import oracle_bindings
    from tiny_dpcpp_nn import cabi as gpu_harness
    from tiny_dpcpp_nn.cabi import ptr
    from tiny_dpcpp_nn import _lib
    from tolerances import BF16, FP16, FP32

    t = gpu_harness.Harness()
    lib = t.lib
    oracle = None
    if not args.no_cpu_baseline:
        oracle = oracle_bindings.Oracle(os.path.join(ROOT, "oracle", "libtnn_oracle.so"))

    K, Wm = args.steps, args.warmup
    ev = lambda: torch.cuda.Event(enable_timing=True)
    out = {}

    if args.workload in ("train", "train_fb", "infer"):
        W, n_hidden = 64, 4
        n_mats = n_hidden + 1
        M = 1 << (args.batch_log2 or 18)
        desc = t.mlp_desc(BF16, W, n_hidden, "relu", "none")
        rng = np.random.default_rng(42)
        lim = np.sqrt(6.0 / (2 * W))
        w = rng.uniform(-lim, lim, (n_mats, W, W)).astype(np.float32)
        gen = torch.Generator(device=t.dev).manual_seed(1234)
        x = (torch.rand((M, W), device=t.dev, generator=gen) * 2 - 1).to(torch.bfloat16)
        # fp32 master weights in the packed parameter layout, as the reference's Python module keeps them
        master = t.pack(FP32, W, n_mats, torch.from_numpy(w.reshape(-1)).to(t.dev))
        pf, pb = t.prepare_packed(desc, master, src_is_fp32=True)

    if args.workload == "train":
        targets = torch.rand((M, W), device=t.dev, generator=gen)
        ws_bytes = lib.tnn_mlp_train_step_workspace_bytes(ctypes.byref(desc), M)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=t.dev)
        loss = torch.zeros(1, device=t.dev)
        m = torch.zeros_like(master)
        v = torch.zeros_like(master)
        s = t.stream()
        d = ctypes.byref(desc)
        # raw HIP events on the stream the kernels go to: one before the call, one the library records between the
        # step's main kernel and the reduction + Adam kernel
        hip = ctypes.CDLL("libamdhip64.so")
        hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        hip.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]

        def hip_event():
            e = ctypes.c_void_p()
            assert hip.hipEventCreate(ctypes.byref(e)) == 0
            return e

        ks, ke = [hip_event() for _ in range(K)], [hip_event() for _ in range(K)]

        def step(i, timed=-1):
            mid = None
            if timed >= 0:
                assert hip.hipEventRecord(ks[timed], s) == 0
                mid = ke[timed]
            rc = lib.tnn_mlp_train_step_l2_adam(d, ptr(pf), ptr(pb), ptr(x), ptr(targets), 1.0, None, ptr(loss), ptr(master), ptr(m), ptr(v),
                                                i + 1, 1e-3, 0.9, 0.99, 1e-15, None, None, M, ptr(ws), ws_bytes, mid, s)
            if rc:
                raise RuntimeError(lib.tnn_last_error())

        for i in range(Wm):
            step(i)
        torch.cuda.synchronize()
        loss0 = float(loss.item())
        e0, e1 = ev(), ev()
        t0 = time.perf_counter()
        e0.record()
        for i in range(K):
            step(Wm + i)
        e1.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ms = e0.elapsed_time(e1) / K
        # a second pass of K steps, each bracketed by HIP events on the launch stream, for the kernel's own duration
        # (kept out of the timed region above: an event between two launches costs about a microsecond)
        for i in range(K):
            step(Wm + K + i, timed=i)
        torch.cuda.synchronize()
        kern_ms = 0.0
        for a, b in zip(ks, ke):
            dt = ctypes.c_float()
            assert hip.hipEventElapsedTime(ctypes.byref(dt), a, b) == 0
            kern_ms += dt.value / K
        flops = 3 * 2 * M * W * W * n_mats  # reference convention: forward + backward-data + dW
        out = {
            "metric": "fused-MLP train & infer samples/s (w64, batch 2^18); % bf16 MFMA peak",
            "value": M / (ms * 1e-3), "unit": "samples/s", "n_gpus": 1, "steps": K, "warmup": Wm, "ms_per_step": ms,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": f"training step: w64, 4 hidden layers (5 matmuls), ReLU/linear, bf16, batch 2^{int(np.log2(M))}, "
                                   "L2 loss, Adam on fp32 masters (BASELINE config 2)", "batch": M},
            "roofline": {"bound": "mfma", "achieved": flops / (kern_ms * 1e-3) / 1e12, "peak": PEAK_MFMA_BF16, "unit": "TFLOP/s",
                         "frac": flops / (kern_ms * 1e-3) / 1e12 / PEAK_MFMA_BF16,
                         "traffic": MEASURED_TRAFFIC_BYTES.get(("train", int(np.log2(M)))),
                         "kernel": "mlp_train_fused_kernel (forward + loss + backward + partial dW)", "kernel_ms": kern_ms,
                         "algorithmic_flops_per_launch": flops},
            "mfma_frac_whole_step": flops / (ms * 1e-3) / 1e12 / PEAK_MFMA_BF16,
            "wall_ms_per_step": wall / K * 1e3,
            "loss_first": loss0, "loss_last": float(loss.item()),
        }
        if oracle is not None:
            out["cpu_baseline"] = cpu_baseline_train(oracle, W, n_mats)

    elif args.workload == "train_fb":
        # The reference's own training step (Trainer::training_step, include/trainer.h:23-46): a forward pass that stores every
        # activation, then a backward pass that returns the weight gradients, the deltas and dL/dx. No loss, no optimizer.
        d = ctypes.byref(desc)
        s = t.stream()
        g = (torch.rand((M, W), device=t.dev, generator=gen) * 2 - 1).to(torch.bfloat16) / M
        interm_f = torch.empty((n_mats + 1, M, W), dtype=torch.bfloat16, device=t.dev)
        interm_b = torch.empty((n_mats, M, W), dtype=torch.bfloat16, device=t.dev)
        dW = torch.empty(n_mats * W * W, dtype=torch.bfloat16, device=t.dev)
        dX = torch.empty_like(x)
        ws_bytes = lib.tnn_mlp_backward_workspace_bytes(d, M)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=t.dev)
        mid = ev()

        def step(timed=False):
            _lib.check(lib.tnn_mlp_forward(d, ptr(pf), ptr(x), ptr(interm_f), M, s))
            if timed:
                mid.record()
            _lib.check(lib.tnn_mlp_backward(d, ptr(pb), ptr(g), ptr(interm_f), ptr(interm_b), ptr(dW), 0, ptr(dX), M, ptr(ws), ws_bytes, s))

        for _ in range(Wm):
            step()
        torch.cuda.synchronize()
        e0, e1 = ev(), ev()
        e0.record()
        for _ in range(K):
            step()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / K
        bwd_ms = 0.0
        for _ in range(10):  # the backward call on its own, outside the timed region
            step(timed=True)
            e1.record()
            torch.cuda.synchronize()
            bwd_ms += mid.elapsed_time(e1) / 10
        flops = 3 * 2 * M * W * W * n_mats
        # bytes of the backward call: dL/dy and n_mats activation matrices in, n_mats delta matrices and dL/dx out
        bwd_bytes = (2 * n_mats + 2) * M * W * 2
        out = {
            "metric": "fused-MLP train & infer samples/s (w64, batch 2^18); % bf16 MFMA peak",
            "value": M / (ms * 1e-3), "unit": "samples/s", "n_gpus": 1, "steps": K, "warmup": Wm, "ms_per_step": ms,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": f"training step as the reference's Trainer runs it: forward_pass with stored activations + backward_pass "
                                   f"(deltas, dW, dL/dx), w64, 4 hidden layers, bf16, batch 2^{int(np.log2(M))}; no loss, no optimizer", "batch": M},
            "roofline": {"bound": "hbm", "achieved": bwd_bytes / (bwd_ms * 1e-3) / 1e9, "peak": PEAK_HBM, "unit": "GB/s",
                         "frac": bwd_bytes / (bwd_ms * 1e-3) / 1e9 / PEAK_HBM, "traffic": MEASURED_TRAFFIC_BYTES.get(("train_fb", int(np.log2(M)))),
                         "kernel": "mlp_backward_fused_kernel (+ train_reduce_kernel)", "kernel_ms": bwd_ms,
                         "algorithmic_bytes_per_launch": bwd_bytes},
            "mfma_frac_whole_step": flops / (ms * 1e-3) / 1e12 / PEAK_MFMA_BF16,
        }
        if oracle is not None:
            out["cpu_baseline"] = cpu_baseline_train(oracle, W, n_mats)

    elif args.workload == "infer":
        y = torch.empty_like(x)
        s = t.stream()
        d = ctypes.byref(desc)
        for _ in range(Wm):
            lib.tnn_mlp_inference(d, ptr(pf), ptr(x), ptr(y), M, s)
        torch.cuda.synchronize()
        e0, e1 = ev(), ev()
        e0.record()
        for _ in range(K):
            lib.tnn_mlp_inference(d, ptr(pf), ptr(x), ptr(y), M, s)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / K
        flops = 2 * M * W * W * n_mats
        bytes_ = 2 * M * W * 2 + n_mats * W * W * 2
        out = {
            "metric": "fused-MLP train & infer samples/s (w64, batch 2^18); % bf16 MFMA peak",
            "value": M / (ms * 1e-3), "unit": "samples/s", "n_gpus": 1, "steps": K, "warmup": Wm, "ms_per_step": ms,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": f"inference: w64, 4 hidden layers (5 matmuls), ReLU/linear, bf16, batch 2^{int(np.log2(M))} (BASELINE config 1 shape)",
                       "batch": M},
            "roofline": {"bound": "hbm", "achieved": bytes_ / (ms * 1e-3) / 1e9, "peak": PEAK_HBM, "unit": "GB/s",
                         "frac": bytes_ / (ms * 1e-3) / 1e9 / PEAK_HBM, "traffic": MEASURED_TRAFFIC_BYTES.get(("infer", int(np.log2(M)))),
                         "kernel": "mlp_forward_kernel (inference)",
                         "kernel_ms": ms, "algorithmic_bytes_per_launch": bytes_},
            "mfma_frac": flops / (ms * 1e-3) / 1e12 / PEAK_MFMA_BF16,
        }
        if oracle is not None:
            out["cpu_baseline"] = cpu_baseline_infer(oracle, W, n_mats)

    elif args.workload == "grid_train":
        # BASELINE config 4: 2-D hash grid -> w64 network with 2 hidden layers, 3 real outputs, one whole optimisation step:
        # encoding, fused network step (forward, L2, backward, dL/d(encoding), Adam on the weights), scatter into the gradient
        # table, Adam on the table's fp32 master with the fp16 table re-rounded
        cfg = dict(n_dims=2, n_levels=16, n_features_per_level=2, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.5)
        W, n_hidden, n_out = 64, 2, 3
        M = 1 << (args.batch_log2 or 18)
        gd = t.grid_desc(cfg, FP16)
        n = t.grid_n_params(gd)
        gen = torch.Generator(device=t.dev).manual_seed(7)
        table_master = torch.rand(n, device=t.dev, generator=gen) * 2e-4 - 1e-4
        table = table_master.to(torch.float16)
        mt, vt = torch.zeros_like(table_master), torch.zeros_like(table_master)
        grad_table = torch.zeros(n, dtype=torch.float16 if args.packed_scatter else torch.float32, device=t.dev)
        x = torch.rand((M, 2), device=t.dev, generator=gen)
        targets = torch.zeros((M, W), device=t.dev)
        targets[:, :n_out] = torch.rand((M, n_out), device=t.dev, generator=gen)
        mdesc = t.mlp_desc(FP16, W, n_hidden, "relu", "none")
        md = ctypes.byref(mdesc)
        rng = np.random.default_rng(42)
        lim = np.sqrt(6.0 / (2 * W))
        w = rng.uniform(-lim, lim, (n_hidden + 1, W, W)).astype(np.float32)
        w[0, 32:, :] = 0
        w[-1, :, n_out:] = 0
        master = t.pack(FP32, W, n_hidden + 1, torch.from_numpy(w.reshape(-1)).to(t.dev))
        pf, pb = t.prepare_packed(mdesc, master, src_is_fp32=True)
        mw, vw = torch.zeros_like(master), torch.zeros_like(master)
        loss = torch.zeros(1, device=t.dev)
        enc = torch.empty((M, W), dtype=torch.float16, device=t.dev)
        d_enc = torch.empty_like(enc)
        ws_bytes = lib.tnn_mlp_train_step_workspace_bytes(md, M)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=t.dev)
        # the loss of the config averages over the 3 real outputs, the fused step over the padded width: the factor W / 3 goes
        # into the loss scale, which also keeps the fp16 gradients clear of the denormal range at this batch size
        loss_scale = 128.0 * W / n_out * (M / 8192)
        s = t.stream()
        g = ctypes.byref(gd)
        hyper = (1e-3, 0.9, 0.99, 1e-15)
        k0, k1 = ev(), ev()

        def step(i, time_scatter=False):
            _lib.check(lib.tnn_grid_forward(g, ptr(x), ptr(table), ptr(enc), FP16, W, M, s))
            _lib.check(lib.tnn_mlp_train_step_l2_adam(md, ptr(pf), ptr(pb), ptr(enc), ptr(targets), loss_scale, None, ptr(loss), ptr(master),
                                                      ptr(mw), ptr(vw), i + 1, *hyper, None, ptr(d_enc), M, ptr(ws), ws_bytes, None, s))
            if time_scatter:
                k0.record()
            if args.packed_scatter:
                _lib.check(lib.tnn_grid_backward_packed(g, ptr(x), ptr(d_enc), FP16, W, ptr(grad_table), 1, M, s))
            else:
                _lib.check(lib.tnn_grid_backward(g, ptr(x), ptr(d_enc), FP16, W, ptr(grad_table), 1, M, s))
            if time_scatter:
                k1.record()
            _lib.check(lib.tnn_adam_step(ptr(table_master), ptr(mt), ptr(vt), ptr(grad_table), FP16 if args.packed_scatter else FP32,
                                         1.0 / loss_scale, n, i + 1, *hyper, ptr(table), FP16, s))

        K = min(K, 50)
        Wm = min(Wm, 5)
        for i in range(Wm):
            step(i)
        torch.cuda.synchronize()
        loss0 = float(loss.item()) * W / n_out  # mean over the real outputs
        e0, e1 = ev(), ev()
        e0.record()
        for i in range(K):
            step(Wm + i)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / K
        scatter_ms = 0.0
        for i in range(10):  # the scatter (fill of the gradient table + atomics) on its own, outside the timed region
            step(Wm + K + i, time_scatter=True)
            torch.cuda.synchronize()
            scatter_ms += k0.elapsed_time(k1) / 10
        # algorithmic bytes of the scatter per point: coordinates + dL/d(encoding) row + read-modify-write of 16 levels x 4 corners x
        # 2 features (4-byte gradients: 1096 B; 2-byte: 584 B)
        gb = 2 if args.packed_scatter else 4
        bpp = 8 + 32 * 2 + 16 * 4 * 2 * gb * 2
        out = {
            "metric": "hash-grid + fused-MLP training samples/s (2-D, 16x2, log2 19; w64, 2 hidden layers; batch 2^18; whole step with both Adam updates)",
            "value": M / (ms * 1e-3), "unit": "samples/s", "n_gpus": 1, "steps": K, "warmup": Wm, "ms_per_step": ms,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": f"2-D hash-grid encoding + w64/2-hidden-layer network, one optimisation step, 2^{int(np.log2(M))} points "
                                   f"(BASELINE config 4; gradient table {'fp16, packed atomics' if args.packed_scatter else 'fp32'})", "batch": M},
            "roofline": {"bound": "hbm", "achieved": bpp * M / (scatter_ms * 1e-3) / 1e9, "peak": PEAK_HBM, "unit": "GB/s",
                         "frac": bpp * M / (scatter_ms * 1e-3) / 1e9 / PEAK_HBM,
                         "traffic": MEASURED_TRAFFIC_BYTES.get(("grid_train_packed" if args.packed_scatter else "grid_train", int(np.log2(M)))),
                         "kernel": "grid_backward_kernel (with the fill of the gradient table in front of it)",
                         "kernel_ms": scatter_ms, "algorithmic_bytes_per_launch": bpp * M},
            "loss_first": loss0, "loss_last": float(loss.item()) * W / n_out,
        }
        if oracle is not None:
            out["cpu_baseline"] = cpu_baseline_grid_train(oracle, cfg, oracle.round(w, FP16))

    else:
        cfg = dict(n_dims=3, n_levels=16, n_features_per_level=2, log2_hashmap_size=22, base_resolution=16, per_level_scale=1.447)
        M = 1 << (args.batch_log2 or 21)
        gd = t.grid_desc(cfg, FP16)
        n = t.grid_n_params(gd)
        gen = torch.Generator(device=t.dev).manual_seed(7)
        table = (torch.rand(n, device=t.dev, generator=gen) * 2e-4 - 1e-4).to(torch.float16)
        x = torch.rand((M, 3), device=t.dev, generator=gen)
        s = t.stream()
        K = min(K, 50)
        if args.workload == "grid":
            o = torch.empty((M, 32), dtype=torch.float16, device=t.dev)
            call = lambda: lib.tnn_grid_forward(ctypes.byref(gd), ptr(x), ptr(table), ptr(o), FP16, 32, M, s)
            bpp = 12 + 16 * 8 * 4 + 32 * 2
        else:
            # BASELINE config 5 whole: the encoding feeds a width-64 network with 3 hidden layers (16 real outputs) in one kernel
            W, n_hidden, n_out = 64, 3, 16
            mdesc = t.mlp_desc(FP16, W, n_hidden, "relu", "none")
            rng = np.random.default_rng(42)
            lim = np.sqrt(6.0 / (2 * W))
            w = rng.uniform(-lim, lim, (n_hidden + 1, W, W)).astype(np.float32)
            w[0, 32:, :] = 0
            w[-1, :, n_out:] = 0
            _, pf, _ = t.prepare(mdesc, w)
            o = torch.empty((M, W), dtype=torch.float16, device=t.dev)
            call = lambda: lib.tnn_grid_mlp_inference(ctypes.byref(gd), ctypes.byref(mdesc), ptr(x), ptr(table), ptr(pf), ptr(o), M, s)
            bpp = 12 + 16 * 8 * 4 + W * 2  # coordinates + gathers + the padded output row; the encoded row stays on chip
        for _ in range(min(Wm, 5)):
            rc = call()
            if rc:
                raise RuntimeError(lib.tnn_last_error())
        torch.cuda.synchronize()
        e0, e1 = ev(), ev()
        e0.record()
        for _ in range(K):
            call()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / K
        grid_only = args.workload == "grid"
        out = {
            "metric": ("hash-grid forward points/s (3-D, 16x2, log2 22, fp16 table, batch 2^21); % HBM peak" if grid_only else
                       "hash-grid + fused-MLP inference points/s (3-D, 16x2, log2 22, fp16; w64, 3 hidden layers; batch 2^21); % HBM peak"),
            "value": M / (ms * 1e-3), "unit": "points/s", "n_gpus": 1, "steps": K, "warmup": min(Wm, 5), "ms_per_step": ms,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": (f"3-D hash-grid encoding forward, 2^{int(np.log2(M))} points (BASELINE config 5 encoding)" if grid_only else
                                    f"3-D hash-grid encoding + w64/3-hidden-layer network inference in one kernel, 2^{int(np.log2(M))} points "
                                    "(BASELINE config 5)"), "batch": M},
            "roofline": {"bound": "hbm", "achieved": bpp * M / (ms * 1e-3) / 1e9, "peak": PEAK_HBM, "unit": "GB/s",
                         "frac": bpp * M / (ms * 1e-3) / 1e9 / PEAK_HBM, "traffic": MEASURED_TRAFFIC_BYTES.get((args.workload, int(np.log2(M)))),
                         "kernel": "grid_forward_kernel" if grid_only else "grid_mlp_inference_kernel",
                         "kernel_ms": ms, "algorithmic_bytes_per_launch": bpp * M},
        }
        if oracle is not None:
            out["cpu_baseline"] = cpu_baseline_grid(oracle, cfg) if grid_only else cpu_baseline_grid_mlp(oracle, cfg, oracle.round(w, FP16))

    if args.copy_calibration:
        n = 64 << 20
        src = torch.ones(n, dtype=torch.float32, device=t.dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            _lib.check(lib.tnn_cast(FP32, ptr(dst), FP32, ptr(src), n, t.stream()))
        torch.cuda.synchronize()

    print(json.dumps(out))


if __name__ == "__main__":
    main()
