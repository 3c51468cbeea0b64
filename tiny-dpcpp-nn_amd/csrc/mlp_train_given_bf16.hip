// The fused training kernels with the loss gradient given by the caller (backward pass with the activations formed again
// on chip), bf16 storage.
#define TNN_TRAIN_GIVEN 1
#include "mlp_train.inc"

namespace tnn {
int fused_given_launch_bf16(const tnn_mlp_desc *d, const FusedPlan &p, const void *wf, const void *wb, const void *x, const void *dLdy, void *dW,
                            int dW_is_fp32, void *dx, size_t M, float *partials, float *loss_partials, hipStream_t s) {
    return launch_fused_w<bf16_t>(d, p, wf, wb, x, static_cast<const float *>(dLdy), 1.0f, nullptr, nullptr, dW, dW_is_fp32, dx, M, partials,
                                  loss_partials, TrainTail{}, s);
}
} // namespace tnn
