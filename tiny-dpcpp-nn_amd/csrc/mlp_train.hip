// Launch plan and dispatch of the fused training step (kernels: mlp_train.inc, compiled per storage type).
#include "mlp_train_shape.h"

#include <atomic>

namespace tnn {

static std::atomic<int> g_meeting_spin_limit{1 << 22};
int meeting_spin_limit() { return g_meeting_spin_limit.load(std::memory_order_relaxed); }

static constexpr size_t kMaxLds = 160 * 1024;

template <int W> static FusedPlan plan_w(int n_mats, size_t M, int n_cu) {
    FusedPlan p;
    typedef TrainShape<W> S;
    p.lds = S::lds_bytes(n_mats);
    // the layer loop is unrolled and the activations of all layers are live in registers: that bounds the depth
    const int max_mats = (W == 64) ? 5 : 6;
    p.supported = n_mats >= 2 && n_mats <= max_mats && p.lds <= kMaxLds;
    const long long n_tiles = ((long long)M + 31) / 32;
    long long g = (n_tiles + S::WAVES - 1) / S::WAVES;
    // The workspace is sized for two workgroups per CU where the shallow narrow networks leave registers for them; the
    // launch asks the runtime how many actually fit and may use fewer.
    const int per_cu = (W <= 32 && n_mats <= 3) ? 2 : 1;
    if (g > (long long)n_cu * per_cu) g = (long long)n_cu * per_cu;
    if (g < 1) g = 1;
    p.grid = (int)g;
    p.partial_bytes = (size_t)p.grid * n_mats * W * W * sizeof(float);
    p.loss_bytes = (((size_t)p.grid * sizeof(float)) + 255) & ~(size_t)255;
    return p;
}

FusedPlan fused_plan(const tnn_mlp_desc *d, size_t M) {
    const DeviceInfo &di = device_info();
    const int n_cu = di.ok ? di.n_cu : 256;
    const int n_mats = d->n_hidden_layers + 1;
    switch (d->width) {
    case 16: return plan_w<16>(n_mats, M, n_cu);
    case 32: return plan_w<32>(n_mats, M, n_cu);
    case 64: return plan_w<64>(n_mats, M, n_cu);
    default: {
        FusedPlan p{};
        p.supported = false;
        return p;
    }
    }
}

// Used by tnn_mlp_train_step_l2: returns TNN_ERR_UNSUPPORTED when the shape has no fused kernel.
int fused_train_step(const tnn_mlp_desc *d, const void *wf, const void *wb, const void *x, const float *targets, float loss_scale,
                     void *y, float *loss_sum, void *dW, int dW_is_fp32, void *dx, size_t M, void *ws, size_t ws_bytes, const TrainTail &tail,
                     hipStream_t s) {
    const FusedPlan p = fused_plan(d, M);
    if (!p.supported) return TNN_ERR_UNSUPPORTED;
    const size_t need = p.partial_bytes + p.loss_bytes + 512;
    if (!ws || ws_bytes < need) return fail(TNN_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", ws_bytes, need);
    uintptr_t base = (reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255;
    float *loss_partials = reinterpret_cast<float *>(base);
    float *partials = reinterpret_cast<float *>(base + p.loss_bytes);
    if (d->dtype == TNN_BF16)
        return fused_train_launch_bf16(d, p, wf, wb, x, targets, loss_scale, y, loss_sum, dW, dW_is_fp32, dx, M, partials, loss_partials, tail, s);
    return fused_train_launch_fp16(d, p, wf, wb, x, targets, loss_scale, y, loss_sum, dW, dW_is_fp32, dx, M, partials, loss_partials, tail, s);
}

int fused_backward(const tnn_mlp_desc *d, const void *wb, const void *dLdy, const void *interm_fwd, void *interm_bwd, void *dW,
                   int dW_is_fp32, void *dx, size_t M, float *partials, size_t partial_bytes, hipStream_t s) {
    if (d->width > 64) return TNN_ERR_UNSUPPORTED;
    if (d->dtype == TNN_BF16) return fused_backward_launch_bf16(d, wb, dLdy, interm_fwd, interm_bwd, dW, dW_is_fp32, dx, M, partials, partial_bytes, s);
    return fused_backward_launch_fp16(d, wb, dLdy, interm_fwd, interm_bwd, dW, dW_is_fp32, dx, M, partials, partial_bytes, s);
}

// 0 when the shape has no fused kernel
size_t fused_train_workspace_bytes(const tnn_mlp_desc *d, size_t M) {
    const FusedPlan p = fused_plan(d, M);
    return p.supported ? p.partial_bytes + p.loss_bytes + 512 : 0;
}

} // namespace tnn

TNN_API int tnn_debug_set_meeting_spin_limit(int iterations, int *previous) {
    if (iterations < 0) return tnn::fail(TNN_ERR_INVALID_ARGUMENT, "the spin limit cannot be negative");
    const int before = tnn::g_meeting_spin_limit.exchange(iterations, std::memory_order_relaxed);
    if (previous) *previous = before;
    return TNN_OK;
}
