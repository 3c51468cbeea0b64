// C entry points of the training step on an encoded input without the encoded matrix: hash-grid encoding, network
// forward, L2 loss, backward pass and Adam on the network's weights (kernels: grid_mlp_train.inc, built once per network
// type), then the scatter of dL/d(encoding) into the table's gradient (grid.hip).
#include "grid_device.h"
#include "mlp_train_shape.h"

namespace tnn {
int grid_mlp_train_launch_bf16(const tnn_grid_desc *g, const tnn_mlp_desc *d, const FusedPlan &p, const GridLevels &lv, const GridParams &gp,
                               const float *x, const float4 *order, const void *table, const void *wf, const void *wb, const float *targets,
                               float loss_scale, void *y, float *loss_sum, void *d_enc, size_t M, float *partials, float *loss_partials,
                               const TrainTail &tail, hipStream_t s);
int grid_mlp_train_launch_fp16(const tnn_grid_desc *g, const tnn_mlp_desc *d, const FusedPlan &p, const GridLevels &lv, const GridParams &gp,
                               const float *x, const float4 *order, const void *table, const void *wf, const void *wb, const float *targets,
                               float loss_scale, void *y, float *loss_sum, void *d_enc, size_t M, float *partials, float *loss_partials,
                               const TrainTail &tail, hipStream_t s);
int grid_mlp_given_launch_bf16(const tnn_grid_desc *g, const tnn_mlp_desc *d, const FusedPlan &p, const GridLevels &lv, const GridParams &gp,
                               const float *x, const float4 *order, const void *table, const void *wf, const void *wb, const void *dLdy,
                               void *dW, int dW_is_fp32, void *d_enc, size_t M, float *partials, float *loss_partials, hipStream_t s);
int grid_mlp_given_launch_fp16(const tnn_grid_desc *g, const tnn_mlp_desc *d, const FusedPlan &p, const GridLevels &lv, const GridParams &gp,
                               const float *x, const float4 *order, const void *table, const void *wf, const void *wb, const void *dLdy,
                               void *dW, int dW_is_fp32, void *d_enc, size_t M, float *partials, float *loss_partials, hipStream_t s);
} // namespace tnn

using namespace tnn;

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// The shapes the one-kernel step is built for: the width-64 network with ReLU and at most four hidden layers (the kernel
// of the plain training step that keeps a workgroup's tiles in LDS), two features per level.
static int train_shape_check(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, size_t M, GridLevels *lv, GridParams *gp, FusedPlan *plan) {
    int rc = check_mlp_desc(mlp);
    if (rc) return rc;
    if ((rc = grid_common(grid, (uint32_t)mlp->width, M, lv, gp))) return rc;
    if (mlp->width != 64 || mlp->activation != TNN_ACT_RELU || grid->n_features_per_level != 2)
        return fail(TNN_ERR_UNSUPPORTED, "fused encoding + training step: built for width 64, ReLU and 2 features per level; run the three calls");
    *plan = fused_plan(mlp, M);
    if (!plan->supported) return fail(TNN_ERR_UNSUPPORTED, "fused encoding + training step: no fused training kernel for this depth; run the three calls");
    return TNN_OK;
}

TNN_API int tnn_grid_mlp_train_supported(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp) {
    GridLevels lv;
    GridParams gp;
    FusedPlan plan;
    return train_shape_check(grid, mlp, 8, &lv, &gp, &plan);
}

TNN_API size_t tnn_grid_mlp_train_step_workspace_bytes(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, size_t M) {
    GridLevels lv;
    GridParams gp;
    FusedPlan plan;
    if (train_shape_check(grid, mlp, M ? M : 8, &lv, &gp, &plan)) return 0;
    // dL/d(encoding) for the scatter, then the partial weight gradients and losses of the workgroups
    return align256(M * 64 * 2) + align256(plan.loss_bytes) + align256(plan.partial_bytes) + 512;
}

TNN_API int tnn_grid_mlp_train_step_l2_adam(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, const float *d_x, const void *d_order,
                                            const void *d_table, void *d_prepared_fwd, void *d_prepared_bwd, const float *d_targets,
                                            float loss_scale, void *d_y, float *d_loss_sum, float *d_master_packed, float *d_m, float *d_v,
                                            int step, float lr, float beta1, float beta2, float eps, void *d_packed_T, float *d_grad_table,
                                            int overwrite, size_t M, void *d_workspace, size_t workspace_bytes, tnn_stream_t stream) {
    GridLevels lv;
    GridParams gp;
    FusedPlan plan;
    int rc = train_shape_check(grid, mlp, M ? M : 8, &lv, &gp, &plan);
    if (rc) return rc;
    if (M == 0 || (M % 8) != 0) return fail(TNN_ERR_INVALID_ARGUMENT, "batch size %zu is not a positive multiple of 8", M);
    if ((!d_x && !d_order) || !d_table || !d_prepared_fwd || !d_prepared_bwd || !d_targets || !d_master_packed || !d_m || !d_v || !d_grad_table)
        return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (reinterpret_cast<uintptr_t>(d_order) & 15) return fail(TNN_ERR_INVALID_ARGUMENT, "d_order must be 16-byte aligned");
    if (loss_scale == 0.0f) return fail(TNN_ERR_INVALID_ARGUMENT, "loss_scale must not be 0");
    if (step < 1) return fail(TNN_ERR_INVALID_ARGUMENT, "step counts from 1");
    const size_t need = tnn_grid_mlp_train_step_workspace_bytes(grid, mlp, M);
    if (!d_workspace || workspace_bytes < need) return fail(TNN_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    hipStream_t s = as_stream(stream);
    uintptr_t base = align256(reinterpret_cast<uintptr_t>(d_workspace));
    void *d_enc_grad = reinterpret_cast<void *>(base);
    base += align256(M * 64 * 2);
    float *loss_partials = reinterpret_cast<float *>(base);
    base += align256(plan.loss_bytes);
    float *partials = reinterpret_cast<float *>(base);

    TrainTail tail;
    tail.use_adam = true;
    tail.adam = make_adam_args(d_master_packed, d_m, d_v, 1.0f / loss_scale, step, lr, beta1, beta2, eps, d_packed_T, d_prepared_fwd, d_prepared_bwd,
                               mlp->width);
    const float4 *order = static_cast<const float4 *>(d_order);
    if (mlp->dtype == TNN_BF16)
        rc = grid_mlp_train_launch_bf16(grid, mlp, plan, lv, gp, d_x, order, d_table, d_prepared_fwd, d_prepared_bwd, d_targets, loss_scale, d_y,
                                        d_loss_sum, d_enc_grad, M, partials, loss_partials, tail, s);
    else
        rc = grid_mlp_train_launch_fp16(grid, mlp, plan, lv, gp, d_x, order, d_table, d_prepared_fwd, d_prepared_bwd, d_targets, loss_scale, d_y,
                                        d_loss_sum, d_enc_grad, M, partials, loss_partials, tail, s);
    if (rc) return rc;
    // dL/d(encoding), in the network's type and at its padded width, into the table's gradient
    if (d_order) return tnn_grid_backward_ordered(grid, d_order, d_enc_grad, mlp->dtype, 64, d_grad_table, overwrite, M, stream);
    return tnn_grid_backward(grid, d_x, d_enc_grad, mlp->dtype, 64, d_grad_table, overwrite, M, stream);
}

TNN_API int tnn_grid_mlp_backward(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, const float *d_x, const void *d_order, const void *d_table,
                                  const void *d_prepared_fwd, const void *d_prepared_bwd, const void *d_dLdy, void *d_dW, int dW_is_fp32,
                                  float *d_grad_table, int overwrite, size_t M, void *d_workspace, size_t workspace_bytes, tnn_stream_t stream) {
    GridLevels lv;
    GridParams gp;
    FusedPlan plan;
    int rc = train_shape_check(grid, mlp, M ? M : 8, &lv, &gp, &plan);
    if (rc) return rc;
    if (M == 0 || (M % 8) != 0) return fail(TNN_ERR_INVALID_ARGUMENT, "batch size %zu is not a positive multiple of 8", M);
    if ((!d_x && !d_order) || !d_table || !d_prepared_fwd || !d_prepared_bwd || !d_dLdy || !d_dW)
        return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (reinterpret_cast<uintptr_t>(d_order) & 15) return fail(TNN_ERR_INVALID_ARGUMENT, "d_order must be 16-byte aligned");
    const size_t need = tnn_grid_mlp_train_step_workspace_bytes(grid, mlp, M);
    if (!d_workspace || workspace_bytes < need) return fail(TNN_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    hipStream_t s = as_stream(stream);
    uintptr_t base = align256(reinterpret_cast<uintptr_t>(d_workspace));
    void *d_enc_grad = reinterpret_cast<void *>(base);
    base += align256(M * 64 * 2);
    float *loss_partials = reinterpret_cast<float *>(base);
    base += align256(plan.loss_bytes);
    float *partials = reinterpret_cast<float *>(base);
    const float4 *order = static_cast<const float4 *>(d_order);
    // without a gradient table the network's gradients are all that is asked for: no dL/d(encoding) leaves the kernel
    void *enc_out = d_grad_table ? d_enc_grad : nullptr;
    if (mlp->dtype == TNN_BF16)
        rc = grid_mlp_given_launch_bf16(grid, mlp, plan, lv, gp, d_x, order, d_table, d_prepared_fwd, d_prepared_bwd, d_dLdy, d_dW, dW_is_fp32, enc_out,
                                        M, partials, loss_partials, s);
    else
        rc = grid_mlp_given_launch_fp16(grid, mlp, plan, lv, gp, d_x, order, d_table, d_prepared_fwd, d_prepared_bwd, d_dLdy, d_dW, dW_is_fp32, enc_out,
                                        M, partials, loss_partials, s);
    if (rc || !d_grad_table) return rc;
    if (d_order) return tnn_grid_backward_ordered(grid, d_order, d_enc_grad, mlp->dtype, 64, d_grad_table, overwrite, M, stream);
    return tnn_grid_backward(grid, d_x, d_enc_grad, mlp->dtype, 64, d_grad_table, overwrite, M, stream);
}
