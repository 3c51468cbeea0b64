// Shape constants and the launch plan of the fused training-step kernel.
#pragma once

#include "adam_update.h"
#include "mlp_tile.h"

namespace tnn {

template <int W> struct TrainShape {
    static constexpr int NK = W / 16;
    static constexpr int NI = (W + 31) / 32;
    static constexpr bool SHARED = (NI * NI >= 4); // dW tiles spread over waves that share all staged rows
    static constexpr int PITCH = W * 2 + 16;       // bytes per staged row (16-byte skew)
    static constexpr int TILE_BYTES = 32 * PITCH;
    static constexpr int WAVES = kTrainThreads / 64;
    static constexpr int CONTROL_BYTES = 64; // behind the staged tiles: the groups' arrival counters and the gave-up flag
    static size_t weight_bytes(int n_mats) { return (size_t)n_mats * NI * NK * 64 * 16; }
    static size_t lds_bytes(int n_mats) {
        const size_t stage = (size_t)WAVES * 2 * TILE_BYTES;
        // end-of-kernel sum over waves that each hold a whole dW: a tree that starts with four slots
        const size_t reduce = SHARED ? 0 : (size_t)4 * n_mats * W * W * 4;
        const size_t main = 2 * weight_bytes(n_mats) + stage + CONTROL_BYTES;
        return main > reduce ? main : reduce;
    }
};

struct FusedPlan {
    bool supported;
    int grid;
    size_t lds;
    size_t partial_bytes; // fp32 [grid][n_mats][W][W]
    size_t loss_bytes;    // fp32 [grid]
};

FusedPlan fused_plan(const tnn_mlp_desc *d, size_t M);

// Iterations a wave waits at a meeting of the waves that share staged tiles before it gives up (tnn_debug_set_meeting_spin_limit).
int meeting_spin_limit();

// per storage type (mlp_train_bf16.hip / mlp_train_fp16.hip)
int fused_train_launch_bf16(const tnn_mlp_desc *d, const FusedPlan &p, const void *wf, const void *wb, const void *x,
                            const float *targets, float loss_scale, void *y, float *loss_sum, void *dW, int dW_is_fp32, void *dx,
                            size_t M, float *partials, float *loss_partials, const TrainTail &tail, hipStream_t s);
int fused_train_launch_fp16(const tnn_mlp_desc *d, const FusedPlan &p, const void *wf, const void *wb, const void *x,
                            const float *targets, float loss_scale, void *y, float *loss_sum, void *dW, int dW_is_fp32, void *dx,
                            size_t M, float *partials, float *loss_partials, const TrainTail &tail, hipStream_t s);

// The same kernels with dL/dy given by the caller (mlp_train_given_*.hip): backward pass with the activations formed again on chip.
int fused_given_launch_bf16(const tnn_mlp_desc *d, const FusedPlan &p, const void *wf, const void *wb, const void *x, const void *dLdy, void *dW,
                            int dW_is_fp32, void *dx, size_t M, float *partials, float *loss_partials, hipStream_t s);
int fused_given_launch_fp16(const tnn_mlp_desc *d, const FusedPlan &p, const void *wf, const void *wb, const void *x, const void *dLdy, void *dW,
                            int dW_is_fp32, void *dx, size_t M, float *partials, float *loss_partials, hipStream_t s);

// Backward pass with the weight gradients in the same kernel (mlp_backward_fused.inc). TNN_ERR_UNSUPPORTED when the shape has
// no such kernel or the workspace holds no partial tile; the caller then runs the separate kernels.
int fused_backward(const tnn_mlp_desc *d, const void *wb, const void *dLdy, const void *interm_fwd, void *interm_bwd, void *dW,
                   int dW_is_fp32, void *dx, size_t M, float *partials, size_t partial_bytes, hipStream_t s);
int fused_backward_launch_bf16(const tnn_mlp_desc *d, const void *wb, const void *dLdy, const void *interm_fwd, void *interm_bwd, void *dW,
                               int dW_is_fp32, void *dx, size_t M, float *partials, size_t partial_bytes, hipStream_t s);
int fused_backward_launch_fp16(const tnn_mlp_desc *d, const void *wb, const void *dLdy, const void *interm_fwd, void *interm_bwd, void *dW,
                               int dW_is_fp32, void *dx, size_t M, float *partials, size_t partial_bytes, hipStream_t s);

} // namespace tnn
