#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X. Prints ONE JSON line.

Default run = the whole metric ("fused-MLP train & infer samples/s, w64, batch 2^18"):
  top level  BASELINE config 2: one training step of the width-64, 4-hidden-layer bf16 fused MLP at batch 2^18 -- forward,
             L2 loss against U[0,1) targets, backward with weight gradients, Adam (lr 1e-3, betas 0.9/0.99, eps 1e-15) on
             fp32 master weights and re-staging of the updated weights for the next step: one tnn_mlp_train_step_l2_adam
             call, two kernel launches
  "infer"    the same network as fused inference at batch 2^18 (BASELINE config 1's shape at the metric's batch size)
  "grid"     BASELINE config 5's encoding: 3-D hash grid forward, 2^21 points (the third target of the north star)
Inputs are resident in HBM before any timed region.

Protocol of every leg: (1) parity of one call against the CPU oracle on the very tensors that are timed (the line carries
`parity_checked` and the measured differences; a failed check ends the run with an error), (2) `prewarm_ms` of untimed
calls so that the clocks are up before the declared warm-up, (3) --warmup untimed steps, (4) --reps repetitions (default 5)
of EXACTLY --steps steps, enqueued back to back on one stream with a HIP event between repetitions and one synchronisation
at each end; `ms_per_step` is the median repetition and `ms_per_step_reps` lists all of them.

--workload train|infer|grid|train_fb|train_w128|grid_mlp|grid_train runs one workload on its own (the form the profiles under profiles/
were collected with); its line has the same top-level fields.
"""
import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tiny-dpcpp-nn_amd"))
sys.path.insert(0, os.path.join(ROOT, "oracle"))  # the checker: parity check and cpu_baseline leg only

PEAK_MFMA_BF16 = 2500.0  # TFLOP/s, dense
PEAK_HBM = 8000.0  # GB/s
METRIC = "fused-MLP train & infer samples/s (w64, batch 2^18); % bf16 MFMA peak"

# HBM-side bytes per launch of each workload's dominant kernel at the default batch sizes, from rocprofv3 counter runs over this
# file (FETCH_SIZE and WRITE_SIZE, one run each, scaled by what the same counter reads for the --copy-calibration kernel:
# x2.000 and x1.000). The summaries with the commands are profiles/mlp_train_fused_kernel.*.txt, profiles/mlp_forward_kernel.*.txt,
# profiles/grid_forward_kernel.*.txt, profiles/grid_mlp_inference_kernel.*.txt and profiles/grid_backward_kernel.*.txt. Not measured live: counters need the profiler.
MEASURED_TRAFFIC_BYTES = {
    ("train", 18): (55469.6 * 2.0 + 20488.0) * 1024,       # the dispatches without dL/dx (the minimum of the run)
    ("infer", 18): (16578.7 * 2.0 + 32787.1) * 1024,
    ("train_fb", 18): (98597.3 * 2.0 + 217115.0) * 1024,  # the backward kernel
    ("grid", 21): (6380144.1 * 2.0 + 132091.7) * 1024,           # points in the caller's order (--no-cell-order)
    ("grid_ordered", 21): (3579269.6 * 2.0 + 131875.3) * 1024,   # points in cell order, the default
    ("grid_mlp", 21): (6610053.5 * 2.0 + 263715.5) * 1024,
    ("grid_mlp_ordered", 21): (3915783.4 * 2.0 + 264728.9) * 1024,
    ("grid_train", 18): (108943.2 * 2.0 + 236762.7) * 1024,  # the scatter kernel; an atomic request counts as a 32-byte write
    ("grid_train_ordered", 18): (248862.1 * 2.0 + 126583.5) * 1024,
    # the whole width-128 step: forward, top launch, four pair launches, reduction with Adam
    ("train_w128", 20): ((138126.3 + 403751.0 + 4 * 393607.4 + 77222.7) * 2.0 + (2098630.8 + 283206.9 + 4 * 229381.6 + 8674.3)) * 1024,
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--reps", type=int, default=5, help="repetitions of --steps timed steps; the median is reported")
    ap.add_argument("--prewarm-ms", type=float, default=300.0,
                    help="untimed calls for this long before the declared warm-up (a fresh process starts at idle clocks)")
    ap.add_argument("--workload", default="all", choices=["all", "train", "train_fb", "train_w128", "infer", "grid", "grid_mlp", "grid_train", "py_infer", "py_train", "py_grid_train", "line_probe"])
    ap.add_argument("--batch-log2", type=int, default=None)
    ap.add_argument("--packed-scatter", action="store_true",
                    help="grid_train only: gradient table in fp16 with one packed atomic per feature pair (tnn_grid_backward_packed)")
    ap.add_argument("--no-cell-order", action="store_true",
                    help="grid and grid_mlp: encode the points as they come instead of ordering the batch by cell in every step")
    ap.add_argument("--unfused", action="store_true",
                    help="grid_train: encoding, network step and scatter as three calls with the encoded matrix in memory")
    ap.add_argument("--push-only-when-changed", action="store_true",
                    help="py_* workloads: switch the modules' push of `params` before every forward off (push_params_every_forward = False)")
    ap.add_argument("--no-extra-legs", action="store_true",
                    help="infer: only the one-buffer leg at the given batch (profiling runs, whose per-kernel averages would otherwise mix three legs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-parity", action="store_true", help="skip the oracle check in front of the timing (profiling runs)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain copy kernel (tnn_cast fp32 -> fp32, 256 MiB read + 256 MiB written per launch) so that "
                         "hardware byte counters collected over this run can be scaled by what they read for a known transfer")
    return ap.parse_args()


# ------------------------------------------------------------------------------------------------------------------
# CPU baselines: the oracle (a port of the reference's arithmetic, OpenMP over rows) on a bounded sample
# ------------------------------------------------------------------------------------------------------------------
def _timed_loop(fn, budget_s):
    fn()
    t0 = time.perf_counter()
    n = 0
    while time.perf_counter() - t0 < budget_s:
        fn()
        n += 1
    return n, time.perf_counter() - t0


def cpu_baseline_train(oracle, W, n_mats, budget_s=12.0, fp16=False):
    import numpy as np
    from tolerances import BF16, FP16

    T = FP16 if fp16 else BF16
    rng = np.random.default_rng(0)
    lim = np.sqrt(6.0 / (2 * W))
    w = oracle.round(rng.uniform(-lim, lim, (n_mats, W, W)), T)
    M = 1 << 14
    x = oracle.round(rng.uniform(-1, 1, (M, W)), T)
    tg = rng.uniform(0, 1, (M, W)).astype(np.float32)

    def step():
        interm = oracle.mlp_forward_T(T, W, n_mats, "relu", "none", w, x)
        _, g = oracle.l2_loss(T, interm[-1], tg, 128.0 if fp16 else 1.0)
        oracle.mlp_backward_T(T, W, n_mats, "relu", "none", w, interm, g, want_dx=False, round_dw=False)

    n, dt = _timed_loop(step, budget_s)
    return {"value": M * n / dt, "unit": "samples/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{n} training steps (forward, L2, backward with dW) of {M} rows each, w{W} / {n_mats - 1} hidden layers, {'fp16' if fp16 else 'bf16'} rounding points, OpenMP over rows"}


def cpu_baseline_infer(oracle, W, n_mats, budget_s=12.0):
    import numpy as np
    from tolerances import BF16

    rng = np.random.default_rng(0)
    lim = np.sqrt(6.0 / (2 * W))
    w = oracle.round(rng.uniform(-lim, lim, (n_mats, W, W)), BF16)
    M = 1 << 15
    x = oracle.round(rng.uniform(-1, 1, (M, W)), BF16)
    n, dt = _timed_loop(lambda: oracle.mlp_forward_T(BF16, W, n_mats, "relu", "none", w, x, store_interm=False), budget_s)
    return {"value": M * n / dt, "unit": "samples/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{n} inference passes of {M} rows, w64 / 4 hidden layers, bf16 rounding points, OpenMP over rows"}


def _cpu_table(oracle, cfg):
    import numpy as np
    from tolerances import FP16

    rng = np.random.default_rng(0)
    off, _, _ = oracle.grid_offsets(cfg["n_dims"], cfg["n_levels"], cfg["log2_hashmap_size"], cfg["base_resolution"], cfg["per_level_scale"])
    n = int(off[-1]) * cfg["n_features_per_level"]
    return rng, n, oracle.round(rng.uniform(-1e-4, 1e-4, n), FP16)


def cpu_baseline_grid(oracle, cfg, budget_s=12.0):
    import numpy as np

    rng, _, table = _cpu_table(oracle, cfg)
    M = 1 << 16
    x = rng.uniform(0, 1, (M, cfg["n_dims"])).astype(np.float32)
    k, dt = _timed_loop(lambda: oracle.grid_forward(cfg, table, x, 32), budget_s)
    return {"value": M * k / dt, "unit": "points/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{k} forward passes of {M} points through the full 162 MiB table, OpenMP over points"}


def cpu_baseline_grid_mlp(oracle, cfg, w, budget_s=12.0):
    import numpy as np
    from tolerances import FP16

    rng, _, table = _cpu_table(oracle, cfg)
    M = 1 << 16
    x = rng.uniform(0, 1, (M, cfg["n_dims"])).astype(np.float32)
    n_mats = w.shape[0]

    def chain():
        enc = oracle.round(oracle.grid_forward(cfg, table, x, 64), FP16)
        return oracle.mlp_forward_T(FP16, 64, n_mats, "relu", "none", w, enc, store_interm=False)

    k, dt = _timed_loop(chain, budget_s)
    return {"value": M * k / dt, "unit": "points/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{k} passes of {M} points: encoding through the full 162 MiB table, then the 4-matrix network, OpenMP over points"}


def cpu_baseline_grid_train(oracle, cfg, w, budget_s=12.0):
    """Config 4's step on the host: encoding, network forward, L2 loss, network backward with dL/d(encoding), scatter into the
    gradient table. (The two Adam updates are elementwise and left out.)"""
    import numpy as np
    from tolerances import FP16

    rng, n, table = _cpu_table(oracle, cfg)
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

    k, dt = _timed_loop(step, budget_s)
    return {"value": M * k / dt, "unit": "samples/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{k} steps of {M} points: encoding, network forward, L2, network backward, scatter into the 7.7 M-entry gradient "
                      "table; OpenMP over points"}


# ------------------------------------------------------------------------------------------------------------------
# GPU timing
# ------------------------------------------------------------------------------------------------------------------
class Timer:
    """Pre-warm, warm-up, then `reps` repetitions of exactly `steps` calls, all enqueued back to back on torch's current
    stream (the stream every launch of this file goes to) with an event between repetitions."""

    def __init__(self, torch, steps, warmup, reps, prewarm_ms):
        self.torch, self.K, self.W, self.reps, self.prewarm_ms = torch, steps, warmup, reps, prewarm_ms
        self.n = 0  # calls made so far (the Adam step number follows it)

    def _call(self, fn, k):
        for _ in range(k):
            fn(self.n)
            self.n += 1

    def run(self, fn, tail=None):
        """tail: further work enqueued directly behind the last repetition, before the synchronisation (a GPU that idles
        for a few milliseconds drops its clocks, and the next hundred launches read 10 % slow)."""
        torch = self.torch
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < self.prewarm_ms:
            self._call(fn, 50)
            torch.cuda.synchronize()
        self._call(fn, self.W)
        torch.cuda.synchronize()
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(self.reps + 1)]
        w0 = time.perf_counter()
        evs[0].record()
        for r in range(self.reps):
            self._call(fn, self.K)
            evs[r + 1].record()
        if tail:
            tail()
        evs[-1].synchronize()
        wall = time.perf_counter() - w0
        torch.cuda.synchronize()
        per_rep = [evs[r].elapsed_time(evs[r + 1]) / self.K for r in range(self.reps)]
        return {"ms": statistics.median(per_rep), "reps_ms": per_rep, "wall_ms": wall / (self.K * self.reps) * 1e3}


class HipEvents:
    """Raw HIP events on the launch stream (one the library records between two kernels of a call cannot be a torch event)."""

    def __init__(self):
        hip = ctypes.CDLL("libamdhip64.so")
        hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        hip.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip = hip

    def create(self):
        e = ctypes.c_void_p()
        assert self.hip.hipEventCreate(ctypes.byref(e)) == 0
        return e

    def record(self, e, stream):
        assert self.hip.hipEventRecord(e, stream) == 0

    def elapsed_ms(self, a, b):
        dt = ctypes.c_float()
        assert self.hip.hipEventElapsedTime(ctypes.byref(dt), a, b) == 0
        return dt.value


def line(metric, unit, dtype, workload, M, tm, K, Wm, args, roofline, extra=None):
    out = {"metric": metric, "value": M / (tm["ms"] * 1e-3), "unit": unit, "n_gpus": 1, "steps": K, "warmup": Wm, "ms_per_step": tm["ms"],
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
           "config": {"workload": workload, "batch": M}, "roofline": roofline, "reps": len(tm["reps_ms"]), "ms_per_step_reps": tm["reps_ms"],
           "prewarm_ms": args.prewarm_ms, "wall_ms_per_step": tm["wall_ms"]}
    if extra:
        out.update(extra)
    return out


class Bench:
    def __init__(self, args):
        import numpy as np
        import torch

        from tiny_dpcpp_nn import _lib, cabi

        self.args, self.np, self.torch, self._lib, self.cabi = args, np, torch, _lib, cabi
        self.t = cabi.Harness()  # raises if the HIP library or the GPU is missing: there is no other path
        self.lib = self.t.lib
        self.oracle = None
        if not (args.no_cpu_baseline and args.no_parity):
            import oracle_bindings
            self.oracle = oracle_bindings.Oracle(os.path.join(ROOT, "oracle", "libtnn_oracle.so"))
        self.K, self.Wm = args.steps, args.warmup

    def timer(self, steps=None, warmup=None):
        return Timer(self.torch, steps or self.K, warmup if warmup is not None else self.Wm, self.args.reps, self.args.prewarm_ms)

    def check(self, rc):
        if rc:
            raise RuntimeError(self.lib.tnn_last_error())

    # --------------------------------------------------------------------------------------------------------------
    def mlp_case(self):
        np, torch, t = self.np, self.torch, self.t
        from tolerances import BF16, FP32
        W, n_hidden = 64, 4
        n_mats = n_hidden + 1
        M = 1 << (self.args.batch_log2 or 18)
        desc = t.mlp_desc(BF16, W, n_hidden, "relu", "none")
        rng = np.random.default_rng(42)
        lim = np.sqrt(6.0 / (2 * W))
        w = rng.uniform(-lim, lim, (n_mats, W, W)).astype(np.float32)
        gen = torch.Generator(device=t.dev).manual_seed(1234)
        x = (torch.rand((M, W), device=t.dev, generator=gen) * 2 - 1).to(torch.bfloat16)
        # fp32 master weights in the packed parameter layout, as the reference's Python module keeps them
        master = t.pack(FP32, W, n_mats, torch.from_numpy(w.reshape(-1)).to(t.dev))
        pf, pb = t.prepare_packed(desc, master, src_is_fp32=True)
        return dict(W=W, n_hidden=n_hidden, n_mats=n_mats, M=M, desc=desc, w=w, gen=gen, x=x, master=master, master0=master.clone(), pf=pf, pb=pb)

    def parity_mlp(self, c, targets):
        """One training step and one inference on the tensors that are timed, against the oracle. Returns the differences."""
        np, torch, t, oracle, lib = self.np, self.torch, self.t, self.oracle, self.lib
        from tiny_dpcpp_nn.cabi import ptr
        from tolerances import BF16, PROPAGATED, assert_close, assert_propagated, bar_report, max_norm_rel
        W, n_mats, M, desc = c["W"], c["n_mats"], c["M"], c["desc"]
        w_T = oracle.round(c["w"], BF16)  # the weights as the kernels see them
        xh, th = t.host(c["x"]), targets.cpu().numpy()
        interm = oracle.mlp_forward_T(BF16, W, n_mats, "relu", "none", w_T, xh)
        res = {}
        y_inf = t.host(t.inference(desc, c["pf"], c["x"]))
        assert_propagated(y_inf, interm[-1], BF16, "bench parity: inference output")
        res["infer_output_max_norm_rel"] = max_norm_rel(y_inf, interm[-1])
        c["y_inference_checked"] = y_inf  # the sub-batch and rotating inference legs compare their rows with these bits
        y, loss, dW, dX = t.train_step_l2(desc, c["pf"], c["pb"], c["x"], targets, 1.0, want_dx=True)
        yh = t.host(y)
        assert_propagated(yh, interm[-1], BF16, "bench parity: training-step output")
        values, grads = oracle.l2_loss(BF16, yh, th, 1.0)
        ref_loss = float(values.astype(np.float64).sum())
        assert abs(float(loss.item()) - ref_loss) <= 1e-4 * ref_loss, "bench parity: loss"
        _, rdW, rdX = oracle.mlp_backward_T(BF16, W, n_mats, "relu", "none", w_T, interm, grads, want_dx=True, round_dw=False)
        dWh, dXh = t.host(dW), t.host(dX)
        # dL/dx is a per-row quantity of natural size 1/M (dL/dy = 2 (y - t) / (M W)); a row whose ReLU mask flipped on a rounding
        # boundary differs in all its elements and is outside any max-norm bound, so the elementwise bar is the check here
        dx_scale = 1.0 / M
        assert_close(dXh, rdX, BF16, "bench parity: dL/dx", scale=dx_scale, frac_ok=PROPAGATED)
        # where the results stand against the STRICT elementwise bar (the end-to-end checks above allow 0.2 % of the elements
        # outside it, none beyond 4x): the counts that actually leave it at this size
        res["strict_bar"] = {"y": bar_report(yh, interm[-1], BF16), "dW": bar_report(dWh, rdW, BF16, scale=float(np.abs(rdW).max())),
                             "dLdx": bar_report(dXh, rdX, BF16, scale=dx_scale)}
        res["dLdx_max_norm_rel"] = max_norm_rel(dXh, rdX)
        res["dW_max_norm_rel"] = max(max_norm_rel(dWh[l], rdW[l]) for l in range(n_mats))
        assert res["dW_max_norm_rel"] < 1e-2, "bench parity: dW"
        assert_propagated(dWh, rdW, BF16, "bench parity: dW", scale=float(np.abs(rdW).max()))
        # the timed entry point: the same step with Adam applied in the reduction, on copies of the optimizer state
        p, m, v = c["master"].clone(), torch.zeros_like(c["master"]), torch.zeros_like(c["master"])
        pf, pb = c["pf"].clone(), c["pb"].clone()
        ws_bytes = lib.tnn_mlp_train_step_workspace_bytes(ctypes.byref(desc), M)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=t.dev)
        l2 = torch.zeros(1, device=t.dev)
        self.check(lib.tnn_mlp_train_step_l2_adam(ctypes.byref(desc), ptr(pf), ptr(pb), ptr(c["x"]), ptr(targets), 1.0, None, ptr(l2), ptr(p), ptr(m),
                                                  ptr(v), 1, 1e-3, 0.9, 0.99, 1e-15, None, None, M, ptr(ws), ws_bytes, None, t.stream()))
        gp = np.concatenate([oracle.pack_and_transpose(dWh[l].ravel(), W) for l in range(n_mats)])
        mh = t.host(c["master"])
        rp, rm, rv = oracle.adam_step(mh, np.zeros_like(mh), np.zeros_like(mh), gp, 1, 1e-3, 0.9, 0.99, 1e-15)
        assert np.allclose(t.host(p), rp, rtol=1e-6, atol=1e-7) and np.allclose(t.host(m), rm, rtol=1e-6, atol=1e-9), "bench parity: Adam"
        assert np.allclose(t.host(v), rv, rtol=1e-6, atol=1e-12) and abs(float(l2.item()) - ref_loss) <= 1e-4 * ref_loss, "bench parity: Adam"
        res["output_max_norm_rel"] = max_norm_rel(yh, interm[-1])
        res["loss_rel"] = abs(float(loss.item()) - ref_loss) / ref_loss
        return res

    def leg_train(self, c, targets):
        np, torch, t, lib = self.np, self.torch, self.t, self.lib
        from tiny_dpcpp_nn.cabi import ptr
        W, n_mats, M, desc = c["W"], c["n_mats"], c["M"], c["desc"]
        ws_bytes = lib.tnn_mlp_train_step_workspace_bytes(ctypes.byref(desc), M)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=t.dev)
        loss = torch.zeros(1, device=t.dev)
        master, pf, pb = c["master"], c["pf"], c["pb"]
        m, v = torch.zeros_like(master), torch.zeros_like(master)
        s, d = t.stream(), ctypes.byref(desc)
        a = (ptr(pf), ptr(pb), ptr(c["x"]), ptr(targets), ptr(loss), ptr(master), ptr(m), ptr(v), ptr(ws))
        hip = HipEvents()

        dLdx = torch.empty_like(c["x"])

        def step(i, mid=None, dx=None):
            rc = lib.tnn_mlp_train_step_l2_adam(d, a[0], a[1], a[2], a[3], 1.0, None, a[4], a[5], a[6], a[7], i + 1, 1e-3, 0.9, 0.99, 1e-15,
                                                None, dx, M, a[8], ws_bytes, mid, s)
            if rc:
                raise RuntimeError(lib.tnn_last_error())

        step(0)
        torch.cuda.synchronize()
        loss0 = float(loss.item())
        timer = self.timer()
        timer.n = 1
        # behind the timed repetitions, a further pass with each step bracketed by HIP events on the launch stream (one
        # recorded here in front of the call, one the library records between the main kernel and the reduction), for the
        # main kernel's own duration; kept out of the timed region: the two events cost about 6 us per step
        nk = 50
        ks, ke = [hip.create() for _ in range(nk)], [hip.create() for _ in range(nk)]

        # ... and the same once more with dL/dx requested (one more product per tile and a batch-sized store)
        kxs, kxe = [hip.create() for _ in range(nk)], [hip.create() for _ in range(nk)]
        xs = [torch.cuda.Event(enable_timing=True) for _ in range(2)]

        def bracketed():
            for i in range(nk):
                hip.record(ks[i], s)
                step(timer.n + i, ke[i])
            for i in range(nk):
                hip.record(kxs[i], s)
                step(timer.n + nk + i, kxe[i], ptr(dLdx))
            xs[0].record()
            for i in range(self.K):
                step(timer.n + 2 * nk + i, None, ptr(dLdx))
            xs[1].record()

        tm = timer.run(step, tail=bracketed)
        kern_ms = statistics.median(hip.elapsed_ms(x, y) for x, y in zip(ks, ke))
        kern_dx_ms = statistics.median(hip.elapsed_ms(x, y) for x, y in zip(kxs, kxe))
        step_dx_ms = xs[0].elapsed_time(xs[1]) / self.K
        # Reference convention (benchmarks/common_benchmarks.h:119-121): forward + backward-data + dW = 3 products per matrix,
        # whether or not dL/dinput is formed. The timed step passes no dL/dx buffer (Trainer::training_step does not either),
        # so the kernel executes 3 * n_mats - 1 of those products; both fractions are given.
        flops = 3 * 2 * M * W * W * n_mats
        executed = (3 * n_mats - 1) * 2 * M * W * W
        lg = int(np.log2(M))
        ach = flops / (kern_ms * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": ach, "peak": PEAK_MFMA_BF16, "unit": "TFLOP/s", "frac": ach / PEAK_MFMA_BF16,
                "traffic": MEASURED_TRAFFIC_BYTES.get(("train", lg)), "kernel": "mlp_train_fused_kernel (forward + loss + backward + partial dW)",
                "kernel_ms": kern_ms, "algorithmic_flops_per_launch": flops, "executed_flops_per_launch": executed,
                "frac_executed": executed / (kern_ms * 1e-3) / 1e12 / PEAK_MFMA_BF16}
        with_dx = {"what": "the same step with dL/dx requested: all 3 * n_mats products executed, dL/dx (M x 64 bf16) stored",
                   "ms_per_step": step_dx_ms, "kernel_ms": kern_dx_ms, "frac": flops / (kern_dx_ms * 1e-3) / 1e12 / PEAK_MFMA_BF16,
                   "mfma_frac_whole_step": flops / (step_dx_ms * 1e-3) / 1e12 / PEAK_MFMA_BF16}
        return line(METRIC, "samples/s", "bf16",
                    f"training step: w64, 4 hidden layers (5 matmuls), ReLU/linear, bf16, batch 2^{lg}, L2 loss, Adam on fp32 masters (BASELINE config 2)",
                    M, tm, self.K, self.Wm, self.args, roof,
                    {"mfma_frac_whole_step": flops / (tm["ms"] * 1e-3) / 1e12 / PEAK_MFMA_BF16,
                     "mfma_frac_whole_step_executed": executed / (tm["ms"] * 1e-3) / 1e12 / PEAK_MFMA_BF16, "with_dLdx": with_dx,
                     "loss_first": loss0, "loss_last": float(loss.item())})

    def leg_infer(self, c, M=None, rotate=1, pf=None):
        """M: rows of the timed call (the first M rows of the case's input). rotate: number of input / output buffer pairs the
        calls cycle through; with enough of them (> 256 MB in all) no call finds its rows in the cache in front of the HBM.
        pf: the prepared weights to run on (the initial ones for a leg whose output is compared with the checked one)."""
        np, torch, t, lib = self.np, self.torch, self.t, self.lib
        from tiny_dpcpp_nn.cabi import ptr
        W, n_mats, desc = c["W"], c["n_mats"], c["desc"]
        M = M or c["M"]
        pf = c["pf"] if pf is None else pf
        xs = [c["x"][:M]] + [c["x"][:M].clone() for _ in range(rotate - 1)]
        ys = [torch.empty_like(xs[0]) for _ in range(rotate)]
        s, d = t.stream(), ctypes.byref(desc)
        a = [(ptr(pf), ptr(x), ptr(y)) for x, y in zip(xs, ys)]

        def step(i):
            b = a[i % rotate]
            if lib.tnn_mlp_inference(d, b[0], b[1], b[2], M, s):
                raise RuntimeError(lib.tnn_last_error())

        tm = self.timer().run(step)
        same = None
        if c.get("y_inference_checked") is not None and pf is not c["pf"]:
            # rows are independent: this leg's output must be, bit for bit, the first M rows of the oracle-checked one
            ref = torch.from_numpy(c["y_inference_checked"][:M]).to(t.dev).to(torch.bfloat16)
            same = all(bool(torch.equal(y.view(torch.int16), ref.view(torch.int16))) for y in ys[: min(rotate, 2)])
            if not same:
                raise AssertionError("bench parity: this inference leg's rows differ from the checked full-batch output")
        flops = 2 * M * W * W * n_mats
        bytes_ = 2 * M * W * 2 + n_mats * W * W * 2
        lg = int(np.log2(M))
        ach = bytes_ / (tm["ms"] * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM, "unit": "GB/s", "frac": ach / PEAK_HBM,
                "traffic": MEASURED_TRAFFIC_BYTES.get(("infer", lg)) if rotate == 1 else None, "kernel": "mlp_forward_kernel (inference)",
                "kernel_ms": tm["ms"], "algorithmic_bytes_per_launch": bytes_, "mfma_frac": flops / (tm["ms"] * 1e-3) / 1e12 / PEAK_MFMA_BF16,
                "buffers_in_rotation_bytes": rotate * 2 * M * W * 2}
        extra = {"mfma_frac": roof["mfma_frac"]}
        if same is not None:
            extra["rows_bit_equal_to_checked_output"] = same
        return line(METRIC, "samples/s", "bf16",
                    f"inference: w64, 4 hidden layers (5 matmuls), ReLU/linear, bf16, batch 2^{lg} (BASELINE config 1" +
                    (")" if lg == 17 else " shape)") +
                    (f"; {rotate} input/output buffer pairs in rotation, {rotate * 2 * M * W * 2 >> 20} MiB in all: no call finds its rows in the "
                     "256 MB cache in front of the HBM" if rotate > 1 else "; one buffer pair (67 MB at 2^18 rows: it stays in that cache between calls)"),
                    M, tm, self.K, self.Wm, self.args, roof, extra)

    # --------------------------------------------------------------------------------------------------------------
    def grid_case(self):
        torch, t = self.torch, self.t
        from tolerances import FP16
        cfg = dict(n_dims=3, n_levels=16, n_features_per_level=2, log2_hashmap_size=22, base_resolution=16, per_level_scale=1.447)
        M = 1 << (self.args.batch_log2 or 21)
        gd = t.grid_desc(cfg, FP16)
        n = t.grid_n_params(gd)
        gen = torch.Generator(device=t.dev).manual_seed(7)
        table = (torch.rand(n, device=t.dev, generator=gen) * 2e-4 - 1e-4).to(torch.float16)
        x = torch.rand((M, 3), device=t.dev, generator=gen)
        return dict(cfg=cfg, M=M, gd=gd, n=n, table=table, x=x)

    def parity_grid(self, g, out_rows, width, what, mlp=None):
        """The first 2^14 points of the timed batch through the oracle: cell selection bit-exact, values within the fp16 bar."""
        np, t, oracle = self.np, self.t, self.oracle
        from tolerances import FP16, assert_close, assert_propagated, max_norm_rel
        n = min(g["M"], 1 << 14)
        xs = g["x"][:n].contiguous()
        assert np.array_equal(t.grid_indices(g["gd"], xs), oracle.grid_indices(g["cfg"], xs.cpu().numpy())), "bench parity: grid indices"
        table = t.host(g["table"])
        if mlp is None:
            ref = oracle.grid_forward(g["cfg"], table, xs.cpu().numpy(), width)
            assert_close(t.host(out_rows[:n]), ref, FP16, what, scale=1e-4)
            return {"grid_indices": "bit-exact", "grid_values_max_norm_rel": max_norm_rel(t.host(out_rows[:n]), ref)}
        enc = oracle.round(oracle.grid_forward(g["cfg"], table, xs.cpu().numpy(), 64), FP16)
        ref = oracle.mlp_forward_T(FP16, 64, mlp.shape[0], "relu", "none", mlp, enc, store_interm=False)
        assert_propagated(t.host(out_rows[:n]), ref, FP16, what, scale=float(np.abs(ref).max()))
        return {"grid_indices": "bit-exact", "output_max_norm_rel": max_norm_rel(t.host(out_rows[:n]), ref)}

    def leg_grid(self, g, fused_mlp=False):
        np, torch, t, lib = self.np, self.torch, self.t, self.lib
        from tiny_dpcpp_nn.cabi import ptr
        from tolerances import FP16
        M, gd = g["M"], g["gd"]
        s = t.stream()
        K, Wm = min(self.K, 50), min(self.Wm, 5)
        w = None
        # every step orders the batch by cell first (tnn_grid_order_points, four small kernels) and then runs the encoding over
        # the ordered records: the ordering is part of the step and inside the timed region
        ob = lib.tnn_grid_order_bytes(ctypes.byref(gd), M)
        order = torch.empty(ob, dtype=torch.uint8, device=t.dev)
        oa = (ctypes.byref(gd), ptr(g["x"]), ptr(order))
        ordered = not self.args.no_cell_order

        def sort_points():
            return lib.tnn_grid_order_points(oa[0], oa[1], M, oa[2], ob, s) if ordered else 0

        if not fused_mlp:
            o = torch.empty((M, 32), dtype=torch.float16, device=t.dev)
            a = (ctypes.byref(gd), ptr(g["x"]), ptr(g["table"]), ptr(o))
            if ordered:
                encode = lambda: lib.tnn_grid_forward_ordered(a[0], oa[2], a[2], a[3], FP16, 32, M, s)
            else:
                encode = lambda: lib.tnn_grid_forward(a[0], a[1], a[2], a[3], FP16, 32, M, s)
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
            a = (ctypes.byref(gd), ctypes.byref(mdesc), ptr(g["x"]), ptr(g["table"]), ptr(pf), ptr(o))
            if ordered:
                encode = lambda: lib.tnn_grid_mlp_inference_ordered(a[0], a[1], oa[2], a[3], a[4], a[5], M, s)
            else:
                encode = lambda: lib.tnn_grid_mlp_inference(a[0], a[1], a[2], a[3], a[4], a[5], M, s)
            bpp = 12 + 16 * 8 * 4 + W * 2  # coordinates + gathers + the padded output row; the encoded row stays on chip

        def call(i):
            return sort_points() or encode()

        self.check(call(0))
        torch.cuda.synchronize()
        parity = None
        if self.oracle is not None and not self.args.no_parity:
            parity = self.parity_grid(g, o, 32, "bench parity: encoding", mlp=self.oracle.round(w, FP16) if fused_mlp else None)
        # behind the timed repetitions: the encoding kernel on its own, between two events, for the roofline of that kernel
        k0 = [torch.cuda.Event(enable_timing=True) for _ in range(10)]
        k1 = [torch.cuda.Event(enable_timing=True) for _ in range(10)]

        def bracketed():
            for i in range(10):
                self.check(sort_points())
                k0[i].record()
                self.check(encode())
                k1[i].record()

        tm = self.timer(K, Wm).run(call, tail=bracketed)
        kern_ms = statistics.median(x.elapsed_time(y) for x, y in zip(k0, k1))
        lg = int(np.log2(M))
        ach = bpp * M / (kern_ms * 1e-3) / 1e9
        name = "grid_mlp" if fused_mlp else "grid"
        roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM, "unit": "GB/s", "frac": ach / PEAK_HBM,
                "traffic": MEASURED_TRAFFIC_BYTES.get((name + ("_ordered" if ordered else ""), lg)),
                "kernel": ("grid_mlp_inference_kernel" if fused_mlp else "grid_forward_kernel") + (" over points in cell order" if ordered else ""),
                "kernel_ms": kern_ms, "algorithmic_bytes_per_launch": bpp * M,
                "frac_whole_step": bpp * M / (tm["ms"] * 1e-3) / 1e9 / PEAK_HBM}
        # A 4-byte gather moves a whole 128-byte line: the bytes the memory side actually moved per launch (`traffic`, from the
        # counters) over the kernel's time, as a fraction of the same peak. `frac` says how far the kernel is from the algorithmic
        # ideal, this one how busy the memory system is.
        if roof["traffic"]:
            roof["frac_lines_moved"] = roof["traffic"] / (kern_ms * 1e-3) / 1e9 / PEAK_HBM
        out = line("hash-grid + fused-MLP inference points/s (3-D, 16x2, log2 22, fp16; w64, 3 hidden layers; batch 2^21); % HBM peak" if fused_mlp else
                   "hash-grid forward points/s (3-D, 16x2, log2 22, fp16 table, batch 2^21); % HBM peak", "points/s", "f16",
                   (f"3-D hash-grid encoding + w64/3-hidden-layer network inference in one kernel, 2^{lg} points (BASELINE config 5)" if fused_mlp else
                    f"3-D hash-grid encoding forward, 2^{lg} points (BASELINE config 5 encoding)") +
                   ("; every step orders the batch by cell, then encodes" if ordered else "; points taken as they come"), M, tm, K, Wm, self.args, roof,
                   {"parity_checked": parity is not None, "parity": parity})
        return out, w

    # --------------------------------------------------------------------------------------------------------------
    def leg_train_w128(self):
        # BASELINE config 3's widest network: width 128, 8 hidden layers, fp16, 2^20 rows. Its nine matrices do not fit one
        # kernel: a forward pass that stores the activations, the top layer's backward launch with the loss in it, then
        # one backward launch per two layers. Parity at this size: tests/test_gpu_mlp.py::test_baseline_config_3_full_size.
        np, torch, t, lib = self.np, self.torch, self.t, self.lib
        from tiny_dpcpp_nn.cabi import ptr
        from tolerances import FP16, FP32
        W, n_hidden = 128, 8
        n_mats = n_hidden + 1
        M = 1 << (self.args.batch_log2 or 20)
        desc = t.mlp_desc(FP16, W, n_hidden, "relu", "none")
        rng = np.random.default_rng(42)
        lim = np.sqrt(6.0 / (2 * W))
        w = rng.uniform(-lim, lim, (n_mats, W, W)).astype(np.float32)
        gen = torch.Generator(device=t.dev).manual_seed(1234)
        x = (torch.rand((M, W), device=t.dev, generator=gen) * 2 - 1).to(torch.float16)
        targets = torch.rand((M, W), device=t.dev, generator=gen)
        master = t.pack(FP32, W, n_mats, torch.from_numpy(w.reshape(-1)).to(t.dev))
        pf, pb = t.prepare_packed(desc, master, src_is_fp32=True)
        m, v = torch.zeros_like(master), torch.zeros_like(master)
        loss = torch.zeros(1, device=t.dev)
        ws_bytes = lib.tnn_mlp_train_step_workspace_bytes(ctypes.byref(desc), M)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=t.dev)
        s, d = t.stream(), ctypes.byref(desc)
        a = (ptr(pf), ptr(pb), ptr(x), ptr(targets), ptr(loss), ptr(master), ptr(m), ptr(v), ptr(ws))

        def step(i):
            if lib.tnn_mlp_train_step_l2_adam(d, a[0], a[1], a[2], a[3], 128.0, None, a[4], a[5], a[6], a[7], i + 1, 1e-3, 0.9, 0.99, 1e-15, None,
                                              None, M, a[8], ws_bytes, None, s):
                raise RuntimeError(lib.tnn_last_error())

        step(0)
        torch.cuda.synchronize()
        loss0 = float(loss.item())
        timer = self.timer()
        timer.n = 1
        tm = timer.run(step)
        flops = 3 * 2 * M * W * W * n_mats
        lg = int(np.log2(M))
        ach = flops / (tm["ms"] * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": ach, "peak": PEAK_MFMA_BF16, "unit": "TFLOP/s", "frac": ach / PEAK_MFMA_BF16,
                "traffic": MEASURED_TRAFFIC_BYTES.get(("train_w128", lg)),
                "kernel": "whole step: mlp_forward_stream_kernel, mlp_layer_backward128_kernel (top layer + loss), "
                          "mlp_layer_pair_backward128_kernel x (n_hidden / 2), train_reduce_kernel (with Adam)",
                "kernel_ms": tm["ms"], "algorithmic_flops_per_launch": flops}
        return line("fused-MLP training samples/s (w128, 8 hidden layers, fp16, batch 2^20); % fp16 MFMA peak", "samples/s", "f16",
                    f"training step: w128, 8 hidden layers (9 matmuls), ReLU/linear, fp16, batch 2^{lg}, L2 loss, Adam on fp32 masters (BASELINE config 3, widest)",
                    M, tm, self.K, self.Wm, self.args, roof, {"loss_first": loss0, "loss_last": float(loss.item())}), W, n_mats

    # --------------------------------------------------------------------------------------------------------------
    def leg_train_fb(self, c):
        # The reference's own training step (Trainer::training_step, include/trainer.h:23-46): a forward pass that stores every
        # activation, then a backward pass that returns the weight gradients, the deltas and dL/dx. No loss, no optimizer.
        np, torch, t, lib, _lib = self.np, self.torch, self.t, self.lib, self._lib
        from tiny_dpcpp_nn.cabi import ptr
        W, n_mats, M, desc = c["W"], c["n_mats"], c["M"], c["desc"]
        d, s = ctypes.byref(desc), t.stream()
        g = (torch.rand((M, W), device=t.dev, generator=c["gen"]) * 2 - 1).to(torch.bfloat16) / M
        interm_f = torch.empty((n_mats + 1, M, W), dtype=torch.bfloat16, device=t.dev)
        interm_b = torch.empty((n_mats, M, W), dtype=torch.bfloat16, device=t.dev)
        dW = torch.empty(n_mats * W * W, dtype=torch.bfloat16, device=t.dev)
        dX = torch.empty_like(c["x"])
        ws_bytes = lib.tnn_mlp_backward_workspace_bytes(d, M)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=t.dev)
        mid, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

        def step(i, timed=False):
            _lib.check(lib.tnn_mlp_forward(d, ptr(c["pf"]), ptr(c["x"]), ptr(interm_f), M, s))
            if timed:
                mid.record()
            _lib.check(lib.tnn_mlp_backward(d, ptr(c["pb"]), ptr(g), ptr(interm_f), ptr(interm_b), ptr(dW), 0, ptr(dX), M, ptr(ws), ws_bytes, s))

        tm = self.timer().run(step)
        bwd = []
        for _ in range(10):  # the backward call on its own, outside the timed region
            step(0, timed=True)
            end.record()
            torch.cuda.synchronize()
            bwd.append(mid.elapsed_time(end))
        bwd_ms = statistics.median(bwd)
        flops = 3 * 2 * M * W * W * n_mats
        bwd_bytes = (2 * n_mats + 2) * M * W * 2  # dL/dy and n_mats activation matrices in, n_mats delta matrices and dL/dx out
        lg = int(np.log2(M))
        ach = bwd_bytes / (bwd_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM, "unit": "GB/s", "frac": ach / PEAK_HBM,
                "traffic": MEASURED_TRAFFIC_BYTES.get(("train_fb", lg)), "kernel": "mlp_backward_fused_kernel (+ train_reduce_kernel)",
                "kernel_ms": bwd_ms, "algorithmic_bytes_per_launch": bwd_bytes}
        return line(METRIC, "samples/s", "bf16",
                    f"training step as the reference's Trainer runs it: forward_pass with stored activations + backward_pass (deltas, dW, dL/dx), "
                    f"w64, 4 hidden layers, bf16, batch 2^{lg}; no loss, no optimizer", M, tm, self.K, self.Wm, self.args, roof,
                    {"mfma_frac_whole_step": flops / (tm["ms"] * 1e-3) / 1e12 / PEAK_MFMA_BF16})

    def leg_grid_train(self):
        # BASELINE config 4: 2-D hash grid -> w64 network with 2 hidden layers, 3 real outputs, one whole optimisation step:
        # encoding, fused network step (forward, L2, backward, dL/d(encoding), Adam on the weights), scatter into the gradient
        # table, Adam on the table's fp32 master with the fp16 table re-rounded
        np, torch, t, lib, _lib, args = self.np, self.torch, self.t, self.lib, self._lib, self.args
        from tiny_dpcpp_nn.cabi import ptr
        from tolerances import FP16, FP32
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
        k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

        # points in cell order (ordered inside the step: a trainer draws new points every step) unless --no-cell-order; the
        # packed scatter has no such route
        ordered = not args.no_cell_order and not args.packed_scatter
        order_bytes = lib.tnn_grid_order_bytes(g, M)
        order = torch.empty(max(order_bytes, 16), dtype=torch.uint8, device=t.dev)

        # one call for encoding + network step + scatter (the encoded matrix never exists) unless --unfused
        fused = not args.unfused and not args.packed_scatter
        fws_bytes = lib.tnn_grid_mlp_train_step_workspace_bytes(g, md, M) if fused else 0
        if fused and fws_bytes == 0:
            raise RuntimeError(lib.tnn_last_error().decode())
        fws = torch.empty(max(fws_bytes, 256) + 256, dtype=torch.uint8, device=t.dev)
        fws_ptr = (fws.data_ptr() + 255) & ~255  # the workspace starts with dL/d(encoding), M x 64 of the network's type

        def fused_step(i, time_scatter=False):
            if ordered:
                _lib.check(lib.tnn_grid_order_points(g, ptr(x), M, ptr(order), order_bytes, s))
            _lib.check(lib.tnn_grid_mlp_train_step_l2_adam(g, md, None if ordered else ptr(x), ptr(order) if ordered else None, ptr(table), ptr(pf),
                                                           ptr(pb), ptr(targets), loss_scale, None, ptr(loss), ptr(master), ptr(mw), ptr(vw), i + 1,
                                                           *hyper, None, ptr(grad_table), 1, M, fws_ptr, fws_bytes, s))
            if time_scatter:  # the scatter once more on its own, from the dL/d(encoding) the call left in its workspace
                k0.record()
                if ordered:
                    _lib.check(lib.tnn_grid_backward_ordered(g, ptr(order), fws_ptr, FP16, W, ptr(grad_table), 1, M, s))
                else:
                    _lib.check(lib.tnn_grid_backward(g, ptr(x), fws_ptr, FP16, W, ptr(grad_table), 1, M, s))
                k1.record()
            _lib.check(lib.tnn_adam_step(ptr(table_master), ptr(mt), ptr(vt), ptr(grad_table), FP32, 1.0 / loss_scale, n, i + 1, *hyper,
                                         ptr(table), FP16, s))

        def step(i, time_scatter=False):
            if fused:
                return fused_step(i, time_scatter)
            if ordered:
                _lib.check(lib.tnn_grid_order_points(g, ptr(x), M, ptr(order), order_bytes, s))
                _lib.check(lib.tnn_grid_forward_ordered(g, ptr(order), ptr(table), ptr(enc), FP16, W, M, s))
            else:
                _lib.check(lib.tnn_grid_forward(g, ptr(x), ptr(table), ptr(enc), FP16, W, M, s))
            _lib.check(lib.tnn_mlp_train_step_l2_adam(md, ptr(pf), ptr(pb), ptr(enc), ptr(targets), loss_scale, None, ptr(loss), ptr(master),
                                                      ptr(mw), ptr(vw), i + 1, *hyper, None, ptr(d_enc), M, ptr(ws), ws_bytes, None, s))
            if time_scatter:
                k0.record()
            if args.packed_scatter:
                _lib.check(lib.tnn_grid_backward_packed(g, ptr(x), ptr(d_enc), FP16, W, ptr(grad_table), 1, M, s))
            elif ordered:
                _lib.check(lib.tnn_grid_backward_ordered(g, ptr(order), ptr(d_enc), FP16, W, ptr(grad_table), 1, M, s))
            else:
                _lib.check(lib.tnn_grid_backward(g, ptr(x), ptr(d_enc), FP16, W, ptr(grad_table), 1, M, s))
            if time_scatter:
                k1.record()
            _lib.check(lib.tnn_adam_step(ptr(table_master), ptr(mt), ptr(vt), ptr(grad_table), FP16 if args.packed_scatter else FP32,
                                         1.0 / loss_scale, n, i + 1, *hyper, ptr(table), FP16, s))

        K, Wm = min(self.K, 50), min(self.Wm, 5)
        step(0)
        torch.cuda.synchronize()
        loss0 = float(loss.item()) * W / n_out  # mean over the real outputs
        timer = self.timer(K, Wm)
        timer.n = 1
        tm = timer.run(step)
        sc = []
        for i in range(10):  # the scatter (fill of the gradient table + atomics) on its own, outside the timed region
            step(timer.n + i, time_scatter=True)
            torch.cuda.synchronize()
            sc.append(k0.elapsed_time(k1))
        scatter_ms = statistics.median(sc)
        # algorithmic bytes of the scatter per point: coordinates + dL/d(encoding) row + read-modify-write of 16 levels x 4 corners x
        # 2 features (4-byte gradients: 1096 B; 2-byte: 584 B)
        gb = 2 if args.packed_scatter else 4
        bpp = 8 + 32 * 2 + 16 * 4 * 2 * gb * 2
        lg = int(np.log2(M))
        ach = bpp * M / (scatter_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM, "unit": "GB/s", "frac": ach / PEAK_HBM,
                "traffic": MEASURED_TRAFFIC_BYTES.get(("grid_train_packed" if args.packed_scatter else ("grid_train_ordered" if ordered else "grid_train"), lg)),
                "kernel": "grid_backward_kernel (with the fill of the gradient table in front of it)" + (" over points in cell order" if ordered else ""),
                "kernel_ms": scatter_ms,
                "algorithmic_bytes_per_launch": bpp * M}
        out = line("hash-grid + fused-MLP training samples/s (2-D, 16x2, log2 19; w64, 2 hidden layers; batch 2^18; whole step with both Adam updates)",
                   "samples/s", "f16",
                   f"2-D hash-grid encoding + w64/2-hidden-layer network, one optimisation step, 2^{lg} points "
                   f"(BASELINE config 4; gradient table {'fp16, packed atomics' if args.packed_scatter else 'fp32'}; "
                   f"{'encoding inside the training kernel' if fused else 'three calls'})", M, tm, K, Wm, args, roof,
                   {"loss_first": loss0, "loss_last": float(loss.item()) * W / n_out})
        return out, cfg, w


# ------------------------------------------------------------------------------------------------------------------
# The drop-in itself: tiny_dpcpp_nn.Network / NetworkWithInputEncoding with torch.optim.Adam, as a user of the reference's Python
# package would run them (the reference's own figures of this kind: samples/benchmark_pytorch.py:24-198). Same shapes as the
# C-ABI legs; each leg also times the C-ABI call that does the same work, in the same process, and reports the ratio.
# ------------------------------------------------------------------------------------------------------------------
def py_legs(b, which):
    import torch

    import tiny_dpcpp_nn as tcnn
    args, t, lib = b.args, b.t, b.lib
    from tiny_dpcpp_nn.cabi import ptr
    dev = "cuda"
    W = 64
    net_cfg = lambda n_hidden: {"otype": "FullyFusedMLP", "activation": "ReLU", "output_activation": "None", "n_neurons": W, "n_hidden_layers": n_hidden}
    every = not args.push_only_when_changed
    push = "params pushed before every forward (the reference's behaviour)" if every else "params pushed only when they changed"

    def timed(fn, steps=None):
        return b.timer(steps).run(lambda i: fn())

    if which == "py_infer":
        M = 1 << (args.batch_log2 or 18)
        net = tcnn.Network(W, W, net_cfg(4), dtype=torch.bfloat16, use_bias=False)
        net.push_params_every_forward = every
        net.eval()
        x = (torch.rand((M, W), device=dev) * 2 - 1).to(torch.bfloat16)
        with torch.no_grad():
            y = net(x)
            tm = timed(lambda: net(x))
        c = b.mlp_case()
        ref = b.leg_infer(c, M=M)
        flops = 2 * M * W * W * 5
        bytes_ = 2 * M * W * 2 + 5 * W * W * 2
        ach = bytes_ / (tm["ms"] * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM, "unit": "GB/s", "frac": ach / PEAK_HBM, "traffic": None,
                "kernel": "whole Python call: Network.forward in eval mode under no_grad", "kernel_ms": tm["ms"], "algorithmic_bytes_per_launch": bytes_,
                "mfma_frac": flops / (tm["ms"] * 1e-3) / 1e12 / PEAK_MFMA_BF16}
        out = line(METRIC, "samples/s", "bf16", f"tiny_dpcpp_nn.Network inference from Python: w64, 4 hidden layers, bf16, batch 2^{M.bit_length() - 1}; {push}",
                   M, tm, b.K, b.Wm, args, roof)
        out.update({"c_abi_ms_per_step": ref["ms_per_step"], "ratio_to_c_abi": tm["ms"] / ref["ms_per_step"], "output_shape": list(y.shape)})
        return out

    if which == "py_train":
        M = 1 << (args.batch_log2 or 18)
        net = tcnn.Network(W, W, net_cfg(4), dtype=torch.bfloat16, use_bias=False)
        net.push_params_every_forward = every
        net.train()
        opt = torch.optim.Adam(net.parameters(), lr=1e-3, betas=(0.9, 0.99), eps=1e-15)
        x = (torch.rand((M, W), device=dev) * 2 - 1).to(torch.bfloat16)
        targets = torch.rand((M, W), device=dev)
        losses = []

        def step():
            opt.zero_grad(set_to_none=True)
            loss = torch.nn.functional.mse_loss(net(x).float(), targets)
            loss.backward()
            opt.step()
            return loss

        losses.append(float(step().detach()))
        tm = timed(step)
        losses.append(float(step().detach()))
        # the module's own share of that step: forward and backward for a dL/dy that is already there (no loss and no optimizer
        # kernels of PyTorch's: its mse_loss alone reads and writes five batch-sized fp32 matrices)
        dy = (torch.rand((M, W), device=dev) / M).to(torch.bfloat16)

        def forward_backward():
            net.params.grad = None
            net(x).backward(dy)

        tm_fb = timed(forward_backward)
        # ... and the same step with PyTorch's one-kernel Adam (fused=True), where the optimizer is one launch instead of a dozen
        opt = torch.optim.Adam(net.parameters(), lr=1e-3, betas=(0.9, 0.99), eps=1e-15, fused=True)
        tm_fused_adam = timed(step)
        c = b.mlp_case()
        ref = b.leg_train(c, torch.rand((c["M"], W), device=t.dev, generator=c["gen"]))
        flops = 3 * 2 * M * W * W * 5
        ach = flops / (tm["ms"] * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": ach, "peak": PEAK_MFMA_BF16, "unit": "TFLOP/s", "frac": ach / PEAK_MFMA_BF16, "traffic": None,
                "kernel": "whole Python step: Network.forward, torch mse_loss, backward (weight gradients with the activations formed again on chip), "
                          "torch.optim.Adam", "kernel_ms": tm["ms"], "algorithmic_flops_per_launch": flops}
        out = line(METRIC, "samples/s", "bf16",
                   f"tiny_dpcpp_nn.Network training step from Python with torch.optim.Adam: w64, 4 hidden layers, bf16, batch 2^{M.bit_length() - 1}, "
                   f"mse_loss in PyTorch; {push}", M, tm, b.K, b.Wm, args, roof)
        out.update({"c_abi_ms_per_step": ref["ms_per_step"], "ratio_to_c_abi": tm["ms"] / ref["ms_per_step"], "loss_first": losses[0], "loss_last": losses[1],
                    "module_forward_backward_ms": tm_fb["ms"], "module_forward_backward_ratio_to_c_abi": tm_fb["ms"] / ref["ms_per_step"],
                    "ms_per_step_with_fused_torch_adam": tm_fused_adam["ms"],
                    "note": "the C-ABI step computes the L2 loss and Adam inside its two kernels; here PyTorch computes them: mse_loss forward and "
                            "backward on a 2^18 x 64 fp32 matrix (about 105 us of its kernels) and torch.optim.Adam (about 45 us of small launches)"})
        return out

    # py_grid_train: BASELINE config 4 through NetworkWithInputEncoding
    M = 1 << (args.batch_log2 or 18)
    enc_cfg = {"otype": "HashGrid", "type": "Hash", "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 19, "base_resolution": 16,
               "per_level_scale": 1.5}
    model = tcnn.NetworkWithInputEncoding(2, 3, net_cfg(2), enc_cfg, dtype=torch.float16, use_bias=False)
    model.network.push_params_every_forward = every
    model.encoding.push_params_every_forward = every
    model.train()
    opt = torch.optim.Adam(model.parameters(), lr=1e-3, betas=(0.9, 0.99), eps=1e-15)
    x = torch.rand((M, 2), device=dev)
    targets = torch.rand((M, 3), device=dev)

    def step():
        opt.zero_grad(set_to_none=True)
        loss = torch.nn.functional.mse_loss(model(x).float(), targets)
        loss.backward()
        opt.step()
        return loss

    K, Wm = min(b.K, 50), min(b.Wm, 5)
    first = float(step().detach())
    tm = b.timer(K, Wm).run(lambda i: step())
    last = float(step().detach())
    ref, _, _ = b.leg_grid_train()
    bpp = 8 + 32 * 2 + 16 * 4 * 2 * 4 * 2  # the scatter's algorithmic bytes per point, as in the grid_train leg
    ach = bpp * M / (tm["ms"] * 1e-3) / 1e9
    roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM, "unit": "GB/s", "frac": ach / PEAK_HBM, "traffic": None,
            "kernel": "whole Python step: fused encoding + network forward, torch mse_loss, fused backward + scatter, torch.optim.Adam over "
                      "network and table", "kernel_ms": tm["ms"], "algorithmic_bytes_per_launch": bpp * M}
    out = line("hash-grid + fused-MLP training samples/s (2-D, 16x2, log2 19; w64, 2 hidden layers; batch 2^18; whole step with both Adam updates)",
               "samples/s", "f16", f"tiny_dpcpp_nn.NetworkWithInputEncoding training step from Python with torch.optim.Adam (BASELINE config 4), "
               f"2^{M.bit_length() - 1} points; {push}", M, tm, K, Wm, args, roof)
    out.update({"c_abi_ms_per_step": ref["ms_per_step"], "ratio_to_c_abi": tm["ms"] / ref["ms_per_step"], "loss_first": first, "loss_last": last})
    return out


def line_probe(b):
    """The ceiling for config 5's gather: random whole 128-byte lines read from buffers of several sizes (one that fits the
    256 MB cache in front of the HBM several times over, the table's own 162 MiB, and 2 GiB, which fits nothing) by 2^21 threads
    reading 32 lines each -- config 5's batch, and the 27-28 lines a point of that batch costs after the cell ordering. Nothing
    but the loads is in the kernel (tnn_probe_line_gather)."""
    import statistics

    torch, t, lib, args = b.torch, b.t, b.lib, b.args
    from tiny_dpcpp_nn.cabi import ptr
    n_threads, per_thread = 1 << (args.batch_log2 or 21), 32
    sink = torch.empty(n_threads, dtype=torch.int32, device=t.dev)
    s = t.stream()
    sizes = {"32 MiB": 32 << 20, "162 MiB (config 5's table)": 42519264 * 2 * 2, "2 GiB": 2 << 30}
    res = {}
    for name, nbytes in sizes.items():
        buf = torch.zeros(nbytes // 4, dtype=torch.int32, device=t.dev)
        n = [0]

        def call(i):
            n[0] += 1
            if lib.tnn_probe_line_gather(ptr(buf), nbytes, n_threads, per_thread, n[0], ptr(sink), s):
                raise RuntimeError(lib.tnn_last_error())

        tm = b.timer(min(b.K, 50), min(b.Wm, 5)).run(call)
        lines = n_threads * per_thread
        res[name] = {"ms": tm["ms"], "lines_per_s": lines / (tm["ms"] * 1e-3), "bytes_of_lines_per_s": lines * 128 / (tm["ms"] * 1e-3)}
        del buf
        torch.cuda.empty_cache()
    key = "162 MiB (config 5's table)"
    ach = res[key]["bytes_of_lines_per_s"] / 1e9
    tm = {"ms": res[key]["ms"], "reps_ms": [res[key]["ms"]], "wall_ms": res[key]["ms"]}
    roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM, "unit": "GB/s", "frac": ach / PEAK_HBM, "traffic": n_threads * per_thread * 128,
            "kernel": "line_gather_probe_kernel (random 128-byte lines, 32 in flight per thread, read-only)", "kernel_ms": res[key]["ms"],
            "algorithmic_bytes_per_launch": n_threads * per_thread * 128}
    out = line("random 128-byte line gathers per second (the ceiling of config 5's hash-grid gather)", "lines/s", "u32",
               f"2^{n_threads.bit_length() - 1} threads x {per_thread} random lines of a buffer", n_threads * per_thread, tm, min(b.K, 50), min(b.Wm, 5), args, roof)
    out["by_buffer_size"] = res
    return out


def sub(leg):
    """A leg as a sub-object of the default line: the fields that differ from the top level."""
    keep = ("value", "unit", "ms_per_step", "ms_per_step_reps", "steps", "warmup", "dtype", "config", "roofline", "mfma_frac", "parity_checked",
            "parity", "cpu_baseline")
    return {k: leg[k] for k in keep if k in leg}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path. Every batch row is independent, so G GPUs would each take "
              "M/G rows with a full copy of the weights and exchange the weight gradients once per step; that is not built. "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    b = Bench(args)
    torch, oracle = b.torch, b.oracle
    from tolerances import FP16
    do_parity = oracle is not None and not args.no_parity
    do_cpu = oracle is not None and not args.no_cpu_baseline
    wl = args.workload

    if wl in ("all", "train", "infer", "train_fb"):
        c = b.mlp_case()
        targets = torch.rand((c["M"], c["W"]), device=b.t.dev, generator=c["gen"])
        parity = b.parity_mlp(c, targets) if (do_parity and wl != "train_fb") else None
    if wl in ("all", "train"):
        out = b.leg_train(c, targets)
        out.update({"parity_checked": parity is not None, "parity": parity})
        if do_cpu:
            out["cpu_baseline"] = cpu_baseline_train(oracle, c["W"], c["n_mats"])
    if wl in ("all", "infer"):
        # the training leg has moved the weights; inference is timed on whatever they are now (its parity ran on the initial ones)
        inf = b.leg_infer(c)
        inf.update({"parity_checked": parity is not None, "parity": parity})
        if do_cpu:
            inf["cpu_baseline"] = cpu_baseline_infer(oracle, c["W"], c["n_mats"], budget_s=6.0 if wl == "all" else 12.0)
        # config 1 at its own batch (2^17) and the 2^18 batch over six buffer pairs (402 MB), both on the initial weights so
        # that their rows can be compared with the oracle-checked output
        extra = {}
        if not args.no_extra_legs:
            pf0 = b.t.prepare_packed(c["desc"], c["master0"], src_is_fp32=True)[0]
            inf17 = b.leg_infer(c, M=1 << 17, pf=pf0)
            inf_hbm = b.leg_infer(c, rotate=6, pf=pf0)
            keep2 = ("value", "ms_per_step", "ms_per_step_reps", "config", "roofline", "mfma_frac", "rows_bit_equal_to_checked_output")
            extra = {"infer_2p17": {k: inf17[k] for k in keep2 if k in inf17}, "infer_hbm": {k: inf_hbm[k] for k in keep2 if k in inf_hbm}}
        if wl == "all":
            out["infer"] = sub(inf)
        else:
            out = inf
        out.update(extra)
    if wl == "train_w128":
        out, W128, n_mats128 = b.leg_train_w128()
        out.update({"parity_checked": False, "parity": None})
        if do_cpu:
            out["cpu_baseline"] = cpu_baseline_train(oracle, W128, n_mats128, fp16=True)
    if wl == "train_fb":
        out = b.leg_train_fb(c)
        if do_cpu:
            out["cpu_baseline"] = cpu_baseline_train(oracle, c["W"], c["n_mats"])
    if wl in ("all", "grid", "grid_mlp"):
        if wl == "all":
            del c, targets
            torch.cuda.empty_cache()
        g = b.grid_case()
        leg, w = b.leg_grid(g, fused_mlp=(wl == "grid_mlp"))
        if do_cpu:
            leg["cpu_baseline"] = (cpu_baseline_grid_mlp(oracle, g["cfg"], oracle.round(w, FP16)) if wl == "grid_mlp" else
                                   cpu_baseline_grid(oracle, g["cfg"], budget_s=6.0 if wl == "all" else 12.0))
        if wl == "all":
            out["grid"] = sub(leg)
        else:
            out = leg
    if wl == "grid_train":
        out, cfg, w = b.leg_grid_train()
        if do_cpu:
            out["cpu_baseline"] = cpu_baseline_grid_train(oracle, cfg, oracle.round(w, FP16))

    if wl in ("py_infer", "py_train", "py_grid_train"):
        out = py_legs(b, wl)
    if wl == "line_probe":
        out = line_probe(b)

    if args.copy_calibration:
        from tiny_dpcpp_nn.cabi import ptr
        from tolerances import FP32
        n = 64 << 20
        src = torch.ones(n, dtype=torch.float32, device=b.t.dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            b._lib.check(b.lib.tnn_cast(FP32, ptr(dst), FP32, ptr(src), n, b.t.stream()))
        torch.cuda.synchronize()

    print(json.dumps(out))


if __name__ == "__main__":
    main()
