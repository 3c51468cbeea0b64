// Fused training-step kernels, bf16 storage.
#include "mlp_backward_fused.inc"
#include "mlp_train.inc"

namespace tnn {
int fused_train_launch_bf16(const tnn_mlp_desc *d, const FusedPlan &p, const void *wf, const void *wb, const void *x,
                            const float *targets, float loss_scale, void *y, float *loss_sum, void *dW, int dW_is_fp32, void *dx,
                            size_t M, float *partials, float *loss_partials, const TrainTail &tail, hipStream_t s) {
    return launch_fused_w<bf16_t>(d, p, wf, wb, x, targets, loss_scale, y, loss_sum, dW, dW_is_fp32, dx, M, partials, loss_partials, tail, s);
}
int fused_backward_launch_bf16(const tnn_mlp_desc *d, const void *wb, const void *dLdy, const void *interm_fwd, void *interm_bwd, void *dW,
                               int dW_is_fp32, void *dx, size_t M, float *partials, size_t partial_bytes, hipStream_t s) {
    return launch_backward_fused_w<bf16_t>(d, wb, dLdy, interm_fwd, interm_bwd, dW, dW_is_fp32, dx, M, partials, partial_bytes, s);
}
} // namespace tnn
