// Fused grid encoding + MLP training step kernels, bf16 network.
#include "grid_mlp_train.inc"

namespace tnn {
int grid_mlp_train_launch_bf16(const tnn_grid_desc *g, const tnn_mlp_desc *d, const FusedPlan &p, const GridLevels &lv, const GridParams &gp,
                               const float *x, const float4 *order, const void *table, const void *wf, const void *wb, const float *targets,
                               float loss_scale, void *y, float *loss_sum, void *d_enc, size_t M, float *partials, float *loss_partials,
                               const TrainTail &tail, hipStream_t s) {
    return launch_grid_train_dp<bf16_t>(g, d, p, lv, gp, x, order, table, wf, wb, targets, loss_scale, y, loss_sum, d_enc, M, partials, loss_partials, tail, s);
}
} // namespace tnn
