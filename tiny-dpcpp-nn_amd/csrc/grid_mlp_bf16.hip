// Fused grid encoding + MLP inference kernels, bf16 network.
#include "grid_mlp.inc"

namespace tnn {
int grid_mlp_launch_bf16(const tnn_grid_desc *g, const GridLevels &lv, const GridParams &gp, const tnn_mlp_desc *mlp, const float *x,
                         const float4 *order, const void *table, const void *wprep, void *y, size_t M, hipStream_t s) {
    return launch_fused_w<bf16_t>(g, lv, gp, mlp, x, order, table, wprep, y, M, s);
}
} // namespace tnn
