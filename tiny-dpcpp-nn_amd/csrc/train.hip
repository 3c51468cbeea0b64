// One training step of the fused MLP against an L2 loss: forward, loss + gradient, backward with
// weight gradients (include/trainer.h:23-46 with include/losses/l2.h:19-40 in between).
#include "mlp_train_shape.h"

#include <mutex>

namespace tnn {

// loss value summed per workgroup, one atomic per workgroup; gradient rounded to T as in l2.h:24
template <typename T>
__global__ void __launch_bounds__(256)
    l2_loss_sum_kernel(const T *__restrict__ pred, const float *__restrict__ target, size_t n, float inv_n, float loss_scale,
                       float *__restrict__ loss_sum, T *__restrict__ grads) {
    __shared__ float red[4];
    float local = 0.0f;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const float diff = (float)pred[i] - target[i];
        local += diff * diff * inv_n;
        grads[i] = (T)as_fp32(loss_scale * 2 * diff * inv_n);
    }
    if (loss_sum) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) local += __shfl_down(local, off, 64);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = local;
        __syncthreads();
        if (threadIdx.x == 0) unsafeAtomicAdd(loss_sum, red[0] + red[1] + red[2] + red[3]);
    }
}

__global__ void zero_scalar_kernel(float *p) { *p = 0.0f; }

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
static size_t unfused_dw_bytes(const tnn_mlp_desc *d) { return (size_t)(d->n_hidden_layers + 1) * d->width * d->width * sizeof(float); }

// mlp_train.hip
int fused_train_step(const tnn_mlp_desc *d, const void *wf, const void *wb, const void *x, const float *targets, float loss_scale,
                     void *y, float *loss_sum, void *dW, int dW_is_fp32, void *dx, size_t M, void *ws, size_t ws_bytes, const TrainTail &tail,
                     hipStream_t s);
size_t fused_train_workspace_bytes(const tnn_mlp_desc *d, size_t M);
// mlp.hip
int forward128_for_training(const tnn_mlp_desc *desc, const void *wprep, const void *x, void *interm_fwd, size_t M, hipStream_t s, bool without_output);
int backward128_from_loss(const tnn_mlp_desc *desc, const void *wprep_bwd, const void *x, const void *interm_fwd, const float *targets, float loss_scale,
                          float *loss_sum, void *dW, int dW_is_fp32, void *dLdx, size_t M, void *workspace, size_t workspace_bytes, hipStream_t s,
                          const void *wprep_fwd_if_no_output, const TrainTail &tail);

} // namespace tnn

using namespace tnn;

TNN_API size_t tnn_mlp_train_step_workspace_bytes(const tnn_mlp_desc *desc, size_t M) {
    if (check_mlp_desc(desc)) return 0;
    const size_t fused = fused_train_workspace_bytes(desc, M);
    if (fused) return fused;
    const size_t mat = M * desc->width * 2;
    // activations, dL/dy, the backward pass's own workspace, and fp32 weight gradients for tnn_mlp_train_step_l2_adam
    return align256((size_t)(desc->n_hidden_layers + 2) * mat) + align256(mat) + align256(tnn_mlp_backward_workspace_bytes(desc, M)) +
           align256(unfused_dw_bytes(desc)) + 512;
}

static int unfused_train_step(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_prepared_bwd, const void *d_x, const float *d_targets,
                              float loss_scale, void *d_y, float *d_loss_sum, void *d_dW, int dW_is_fp32, void *d_dLdx, size_t M, void *d_workspace,
                              const TrainTail &tail, tnn_stream_t stream);

TNN_API int tnn_mlp_train_step_l2(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_prepared_bwd,
                                  const void *d_x, const float *d_targets, float loss_scale, void *d_y, float *d_loss_sum,
                                  void *d_dW, int dW_is_fp32, void *d_dLdx, size_t M, void *d_workspace,
                                  size_t workspace_bytes, tnn_stream_t stream) {
    int rc = check_mlp_desc(desc);
    if (rc) return rc;
    if (!d_prepared_fwd || !d_prepared_bwd || !d_x || !d_targets || !d_dW) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (loss_scale == 0.0f) return fail(TNN_ERR_INVALID_ARGUMENT, "loss_scale must not be 0");
    const size_t need = tnn_mlp_train_step_workspace_bytes(desc, M);
    if (!d_workspace || workspace_bytes < need)
        return fail(TNN_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    hipStream_t s = as_stream(stream);
    if (M == 0 || (M % 8) != 0) return fail(TNN_ERR_INVALID_ARGUMENT, "batch size %zu is not a positive multiple of 8", M);
    // shapes with a fused kernel never touch device memory with activations or deltas
    rc = fused_train_step(desc, d_prepared_fwd, d_prepared_bwd, d_x, d_targets, loss_scale, d_y, d_loss_sum, d_dW, dW_is_fp32, d_dLdx, M,
                          d_workspace, workspace_bytes, TrainTail{}, s);
    if (rc != TNN_ERR_UNSUPPORTED) return rc;
    return unfused_train_step(desc, d_prepared_fwd, d_prepared_bwd, d_x, d_targets, loss_scale, d_y, d_loss_sum, d_dW, dW_is_fp32, d_dLdx, M, d_workspace,
                              TrainTail{}, stream);
}

// Wider / deeper networks than the fused kernel takes: forward, loss and backward as separate kernels over workspace matrices
// (arguments checked by the caller, the workspace at least tnn_mlp_train_step_workspace_bytes). `tail` with Adam: width 128 only.
static int unfused_train_step(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_prepared_bwd, const void *d_x, const float *d_targets,
                              float loss_scale, void *d_y, float *d_loss_sum, void *d_dW, int dW_is_fp32, void *d_dLdx, size_t M, void *d_workspace,
                              const TrainTail &tail, tnn_stream_t stream) {
    int rc;
    hipStream_t s = as_stream(stream);
    const int W = desc->width, n_mats = desc->n_hidden_layers + 1;
    const size_t mat = M * W * 2;
    uintptr_t base = align256(reinterpret_cast<uintptr_t>(d_workspace));
    void *interm_fwd = reinterpret_cast<void *>(base);
    base += align256((size_t)(n_mats + 1) * mat);
    void *dLdy = reinterpret_cast<void *>(base);
    base += align256(mat);
    void *bwd_ws = reinterpret_cast<void *>(base);
    const size_t bwd_ws_bytes = align256(tnn_mlp_backward_workspace_bytes(desc, M));

    // width 128 when nobody asks for the network's output: the forward pass ends at the last hidden layer and the backward
    // pass's first launch forms the output again on chip (one matrix less to write and to read)
    const bool no_output = W == 128 && !d_y && desc->n_hidden_layers >= 2;
    if ((rc = (W == 128 ? forward128_for_training(desc, d_prepared_fwd, d_x, interm_fwd, M, s, no_output) : tnn_mlp_forward(desc, d_prepared_fwd, d_x, interm_fwd, M, stream)))) return rc;
    const void *y = static_cast<const char *>(interm_fwd) + (size_t)n_mats * mat;
    if (d_y && hipMemcpyAsync(d_y, y, mat, hipMemcpyDeviceToDevice, s) != hipSuccess) return fail(TNN_ERR_HIP, "copy of the network output failed");
    const size_t n = M * W;
    // width 128: the loss is part of the backward pass's first launch (dL/dy is never written), its sum and, when asked for,
    // Adam are part of the reduction that ends the pass
    if (W == 128) return backward128_from_loss(desc, d_prepared_bwd, d_x, interm_fwd, d_targets, loss_scale, d_loss_sum, d_dW, dW_is_fp32, d_dLdx, M, bwd_ws,
                                               bwd_ws_bytes, s, no_output ? d_prepared_fwd : nullptr, tail);
    if (d_loss_sum) TNN_LAUNCH(zero_scalar_kernel, dim3(1), dim3(1), 0, s, d_loss_sum);
    size_t blocks = (n + 256 * 8 - 1) / (256 * 8);
    if (blocks > 2048) blocks = 2048;
    const float inv_n = 1.0f / (float)n;
    if (desc->dtype == TNN_BF16)
        TNN_LAUNCH((l2_loss_sum_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, s, (const bf16_t *)y, d_targets, n, inv_n,
                           loss_scale, d_loss_sum, (bf16_t *)dLdy);
    else
        TNN_LAUNCH((l2_loss_sum_kernel<fp16_t>), dim3((unsigned)blocks), dim3(256), 0, s, (const fp16_t *)y, d_targets, n, inv_n,
                           loss_scale, d_loss_sum, (fp16_t *)dLdy);
    if ((rc = check_launch("l2_loss_sum_kernel"))) return rc;
    return tnn_mlp_backward(desc, d_prepared_bwd, dLdy, interm_fwd, nullptr, d_dW, dW_is_fp32, d_dLdx, M, bwd_ws, bwd_ws_bytes, stream);
}

TNN_API int tnn_mlp_train_step_l2_adam(const tnn_mlp_desc *desc, void *d_prepared_fwd, void *d_prepared_bwd, const void *d_x,
                                       const float *d_targets, float loss_scale, void *d_y, float *d_loss_sum, float *d_master_packed,
                                       float *d_m, float *d_v, int step, float lr, float beta1, float beta2, float eps,
                                       void *d_packed_T, void *d_dLdx, size_t M, void *d_workspace, size_t workspace_bytes,
                                       void *main_kernel_done_event, tnn_stream_t stream) {
    int rc = check_mlp_desc(desc);
    if (rc) return rc;
    if (!d_prepared_fwd || !d_prepared_bwd || !d_x || !d_targets || !d_master_packed || !d_m || !d_v)
        return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (loss_scale == 0.0f) return fail(TNN_ERR_INVALID_ARGUMENT, "loss_scale must not be 0");
    if (step < 1) return fail(TNN_ERR_INVALID_ARGUMENT, "step counts from 1");
    const size_t need = tnn_mlp_train_step_workspace_bytes(desc, M);
    if (!d_workspace || workspace_bytes < need)
        return fail(TNN_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    if (M == 0 || (M % 8) != 0) return fail(TNN_ERR_INVALID_ARGUMENT, "batch size %zu is not a positive multiple of 8", M);
    hipStream_t s = as_stream(stream);
    TrainTail tail;
    tail.use_adam = true;
    tail.adam = make_adam_args(d_master_packed, d_m, d_v, 1.0f / loss_scale, step, lr, beta1, beta2, eps, d_packed_T, d_prepared_fwd,
                               d_prepared_bwd, desc->width);
    tail.main_done = static_cast<hipEvent_t>(main_kernel_done_event);
    rc = fused_train_step(desc, d_prepared_fwd, d_prepared_bwd, d_x, d_targets, loss_scale, d_y, d_loss_sum, nullptr, 1, d_dLdx, M,
                          d_workspace, workspace_bytes, tail, s);
    if (rc != TNN_ERR_UNSUPPORTED) return rc;
    // width 128: separate kernels, the update inside the reduction that ends the backward pass (no gradient tensor)
    if (desc->width == 128)
        return unfused_train_step(desc, d_prepared_fwd, d_prepared_bwd, d_x, d_targets, loss_scale, d_y, d_loss_sum, nullptr, 1, d_dLdx, M, d_workspace, tail,
                                  stream);
    // other shapes without a fused kernel: the separate step, then the separate update, over gradients kept in the workspace
    const uintptr_t end = reinterpret_cast<uintptr_t>(d_workspace) + workspace_bytes;
    float *dW = reinterpret_cast<float *>((end - unfused_dw_bytes(desc)) & ~(uintptr_t)255);
    // (the step lays its matrices out from the front of the workspace and stays clear of this tail)
    if ((rc = tnn_mlp_train_step_l2(desc, d_prepared_fwd, d_prepared_bwd, d_x, d_targets, loss_scale, d_y, d_loss_sum, dW, 1, d_dLdx, M,
                                    d_workspace, workspace_bytes, stream)))
        return rc;
    if (tail.main_done && hipEventRecord(tail.main_done, s) != hipSuccess) return fail(TNN_ERR_HIP, "hipEventRecord failed");
    return tnn_mlp_adam_update(desc, d_master_packed, d_m, d_v, dW, 1.0f / loss_scale, step, lr, beta1, beta2, eps, d_packed_T,
                               d_prepared_fwd, d_prepared_bwd, stream);
}

TNN_API int tnn_mlp_backward_recompute_supported(const tnn_mlp_desc *desc) {
    int rc = check_mlp_desc(desc);
    if (rc) return rc;
    if (!fused_plan(desc, 8).supported) return fail(TNN_ERR_UNSUPPORTED, "no fused training kernel for width %d with %d matrices", desc->width, desc->n_hidden_layers + 1);
    return TNN_OK;
}

TNN_API int tnn_mlp_backward_recompute(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_prepared_bwd, const void *d_x,
                                       const void *d_dLdy, void *d_dW, int dW_is_fp32, void *d_dLdx, size_t M, void *d_workspace,
                                       size_t workspace_bytes, tnn_stream_t stream) {
    int rc = tnn_mlp_backward_recompute_supported(desc);
    if (rc) return rc;
    if (!d_prepared_fwd || !d_prepared_bwd || !d_x || !d_dLdy || !d_dW) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (M == 0 || (M % 8) != 0) return fail(TNN_ERR_INVALID_ARGUMENT, "batch size %zu is not a positive multiple of 8", M);
    const FusedPlan p = fused_plan(desc, M);
    const size_t need = p.partial_bytes + p.loss_bytes + 512;
    if (!d_workspace || workspace_bytes < need) return fail(TNN_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    const uintptr_t base = align256(reinterpret_cast<uintptr_t>(d_workspace));
    float *loss_partials = reinterpret_cast<float *>(base);
    float *partials = reinterpret_cast<float *>(base + p.loss_bytes);
    hipStream_t s = as_stream(stream);
    if (desc->dtype == TNN_BF16)
        return fused_given_launch_bf16(desc, p, d_prepared_fwd, d_prepared_bwd, d_x, d_dLdy, d_dW, dW_is_fp32, d_dLdx, M, partials, loss_partials, s);
    return fused_given_launch_fp16(desc, p, d_prepared_fwd, d_prepared_bwd, d_x, d_dLdy, d_dW, dW_is_fp32, d_dLdx, M, partials, loss_partials, s);
}

// ------------------------------------------------------------------------------------------------
// The training step for callers that cannot allocate device memory (code under graph capture, serving loops,
// harnesses that forbid hipMalloc): the partial weight gradients and partial losses go to a fixed array in
// device memory that every GPU using this library holds until the process ends.
// ------------------------------------------------------------------------------------------------
namespace tnn {

constexpr size_t kStaticScratchBytes = TNN_MLP_TRAIN_STEP_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device. In host code the array's name is only a handle for
// hipGetSymbolAddress; each device has its own copy at its own address, resolved once per device.
static int static_scratch(void **out) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void *addr[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return fail(TNN_ERR_HIP, "no current HIP device");
    }
    std::lock_guard<std::mutex> lock(mu);
    if (!addr[dev]) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            return fail(TNN_ERR_HIP, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
        }
        addr[dev] = p;
    }
    *out = addr[dev];
    return TNN_OK;
}

} // namespace tnn

TNN_API size_t tnn_mlp_train_step_l2_static_max_bytes(void) { return kStaticScratchBytes; }

TNN_API int tnn_mlp_train_step_l2_static(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_prepared_bwd,
                                         const void *d_x, const float *d_targets, float loss_scale, void *d_y, float *d_loss_sum,
                                         void *d_dW, int dW_is_fp32, void *d_dLdx, size_t M, tnn_stream_t stream) {
    int rc = check_mlp_desc(desc);
    if (rc) return rc;
    const size_t need = tnn_mlp_train_step_workspace_bytes(desc, M);
    if (need > kStaticScratchBytes)
        return fail(TNN_ERR_WORKSPACE,
                    "this shape and batch size need %zu bytes of scratch memory, the static buffer holds %zu: use "
                    "tnn_mlp_train_step_l2 with a workspace of the caller's",
                    need, kStaticScratchBytes);
    void *ws = nullptr;
    if ((rc = static_scratch(&ws))) return rc;
    // Nothing in the buffer has to start at zero: every workgroup overwrites its own partials before the reduction
    // reads them, and the separate-kernel route writes every matrix before it reads it.
    return tnn_mlp_train_step_l2(desc, d_prepared_fwd, d_prepared_bwd, d_x, d_targets, loss_scale, d_y, d_loss_sum, d_dW, dW_is_fp32,
                                 d_dLdx, M, ws, kStaticScratchBytes, stream);
}
