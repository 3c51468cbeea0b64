// Grid encoding + fused network backward pass for a loss gradient given by the caller, fp16 network.
#define TNN_TRAIN_GIVEN 1
#include "grid_mlp_train.inc"

namespace tnn {
int grid_mlp_given_launch_fp16(const tnn_grid_desc *g, const tnn_mlp_desc *d, const FusedPlan &p, const GridLevels &lv, const GridParams &gp,
                               const float *x, const float4 *order, const void *table, const void *wf, const void *wb, const void *dLdy,
                               void *dW, int dW_is_fp32, void *d_enc, size_t M, float *partials, float *loss_partials, hipStream_t s) {
    TrainTail tail;
    tail.dW = dW;
    tail.dW_is_fp32 = dW_is_fp32;
    return launch_grid_train_dp<fp16_t>(g, d, p, lv, gp, x, order, table, wf, wb, static_cast<const float *>(dLdy), 1.0f, nullptr, nullptr, d_enc, M,
                                        partials, loss_partials, tail, s);
}
} // namespace tnn
