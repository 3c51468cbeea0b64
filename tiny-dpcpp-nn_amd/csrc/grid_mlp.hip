// C entry point of the fused grid encoding + MLP inference (kernels: grid_mlp.inc, built once per network type).
#include "grid_device.h"
#include "mlp_tile.h"

namespace tnn {
int grid_mlp_launch_bf16(const tnn_grid_desc *g, const GridLevels &lv, const GridParams &gp, const tnn_mlp_desc *mlp, const float *x,
                         const float4 *order, const void *table, const void *wprep, void *y, size_t M, hipStream_t s);
int grid_mlp_launch_fp16(const tnn_grid_desc *g, const GridLevels &lv, const GridParams &gp, const tnn_mlp_desc *mlp, const float *x,
                         const float4 *order, const void *table, const void *wprep, void *y, size_t M, hipStream_t s);
} // namespace tnn

using namespace tnn;

// bytes of LDS the fused kernel asks for: the prepared weights and the per-level constants behind them
static size_t fused_lds_bytes(const tnn_mlp_desc *mlp) { return tnn_mlp_prepared_bytes(mlp) + TNN_GRID_MAX_LEVELS * sizeof(LevelConst); }

static int fused_shape_check(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, size_t M, GridLevels *lv, GridParams *gp) {
    int rc = check_mlp_desc(mlp);
    if (rc) return rc;
    if ((rc = grid_common(grid, (uint32_t)mlp->width, M, lv, gp))) return rc;
    const DeviceInfo &di = device_info();
    if (!di.ok) return fail(TNN_ERR_HIP, "no usable HIP device");
    if (fused_lds_bytes(mlp) > di.max_lds)
        return fail(TNN_ERR_UNSUPPORTED, "fused encoding + network: the weights (%zu bytes with the level constants) do not fit LDS; run the two calls",
                    fused_lds_bytes(mlp));
    return TNN_OK;
}

TNN_API int tnn_grid_mlp_supported(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp) {
    GridLevels lv;
    GridParams gp;
    return fused_shape_check(grid, mlp, 8, &lv, &gp);
}

static int grid_mlp_any(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, const float *d_x, const void *d_order, const void *d_table,
                        const void *d_prepared_fwd, void *d_y, size_t M, tnn_stream_t stream) {
    GridLevels lv;
    GridParams gp;
    int rc = fused_shape_check(grid, mlp, M ? M : 8, &lv, &gp);
    if (rc) return rc;
    // include/network/SwiftNetMLP.h:293-300: the batch must be a multiple of 8
    if (M == 0 || (M % 8) != 0) return fail(TNN_ERR_INVALID_ARGUMENT, "batch size %zu is not a positive multiple of 8", M);
    if ((!d_x && !d_order) || !d_table || !d_prepared_fwd || !d_y) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (reinterpret_cast<uintptr_t>(d_order) & 15) return fail(TNN_ERR_INVALID_ARGUMENT, "d_order must be 16-byte aligned");
    hipStream_t s = as_stream(stream);
    const float4 *order = static_cast<const float4 *>(d_order);
    if (mlp->dtype == TNN_BF16) return grid_mlp_launch_bf16(grid, lv, gp, mlp, d_x, order, d_table, d_prepared_fwd, d_y, M, s);
    return grid_mlp_launch_fp16(grid, lv, gp, mlp, d_x, order, d_table, d_prepared_fwd, d_y, M, s);
}

TNN_API int tnn_grid_mlp_inference(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, const float *d_x, const void *d_table,
                                   const void *d_prepared_fwd, void *d_y, size_t M, tnn_stream_t stream) {
    if (!d_x) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    return grid_mlp_any(grid, mlp, d_x, nullptr, d_table, d_prepared_fwd, d_y, M, stream);
}

TNN_API int tnn_grid_mlp_inference_ordered(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, const void *d_order, const void *d_table,
                                           const void *d_prepared_fwd, void *d_y, size_t M, tnn_stream_t stream) {
    if (!d_order) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    return grid_mlp_any(grid, mlp, nullptr, d_order, d_table, d_prepared_fwd, d_y, M, stream);
}
