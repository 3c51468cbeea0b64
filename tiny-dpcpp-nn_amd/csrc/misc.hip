// Error reporting, weight-layout permutations, L2 loss and the Adam step.
#include "tnn_internal.h"
#include "adam_update.h"

#include <cstring>

namespace tnn {

char *error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return status;
}

int check_launch(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(TNN_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
    return TNN_OK;
}

int check_mlp_desc(const tnn_mlp_desc *d) {
    if (!d) return fail(TNN_ERR_INVALID_ARGUMENT, "desc is NULL");
    if (d->dtype != TNN_BF16 && d->dtype != TNN_FP16)
        return fail(TNN_ERR_UNSUPPORTED, "dtype %d: only bf16 and fp16 networks exist", d->dtype);
    // include/network/Network.h:160-161
    if (!valid_width(d->width))
        return fail(TNN_ERR_INVALID_ARGUMENT, "Network width has to be a power of 2 between 16 and 128 (got %d)", d->width);
    // include/network/Network.h:154-158
    if (d->n_hidden_layers < 1)
        return fail(TNN_ERR_INVALID_ARGUMENT, "n_hidden_layers is %d but must be >= 1", d->n_hidden_layers);
    // include/network/SwiftNetMLP.h:276-290
    if (!valid_act(d->activation) || !valid_act(d->output_activation))
        return fail(TNN_ERR_UNSUPPORTED, "activation %d / output activation %d: only None, ReLU and Sigmoid are supported",
                    d->activation, d->output_activation);
    return TNN_OK;
}

enum PermuteOp { OP_PACK, OP_UNPACK, OP_PACKED_TRANSPOSE, OP_PACK_AND_TRANSPOSE };

template <typename T> __global__ void permute_kernel(const T *__restrict__ src, T *__restrict__ dst, int W, int n_mats, int op) {
    const int per = W * W;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= per * n_mats) return;
    const int m = idx / per, e = idx % per;
    const int i = e / W, j = e % W;
    const T *s = src + (size_t)m * per;
    T *d = dst + (size_t)m * per;
    switch (op) {
    case OP_PACK: d[packed_coord(i, j, W)] = s[e]; break;
    case OP_UNPACK: d[e] = s[packed_coord(i, j, W)]; break;
    case OP_PACKED_TRANSPOSE: d[packed_coord(i, j, W)] = s[packed_coord(j, i, W)]; break;
    case OP_PACK_AND_TRANSPOSE: d[packed_coord(i, j, W)] = s[j * W + i]; break;
    }
}

static int launch_permute(int dtype, int W, int n_mats, const void *src, void *dst, int op, hipStream_t s) {
    if (dtype != TNN_BF16 && dtype != TNN_FP16 && dtype != TNN_FP32) return fail(TNN_ERR_UNSUPPORTED, "dtype %d", dtype);
    if (!valid_width(W)) return fail(TNN_ERR_INVALID_ARGUMENT, "width %d", W);
    if (n_mats < 1 || !src || !dst) return fail(TNN_ERR_INVALID_ARGUMENT, "bad arguments");
    if (src == dst) return fail(TNN_ERR_INVALID_ARGUMENT, "in-place permutation is not supported");
    const int total = W * W * n_mats;
    if (dtype == TNN_FP32)
        TNN_LAUNCH((permute_kernel<float>), dim3((total + 255) / 256), dim3(256), 0, s, (const float *)src, (float *)dst,
                           W, n_mats, op);
    else
        TNN_LAUNCH((permute_kernel<uint16_t>), dim3((total + 255) / 256), dim3(256), 0, s, (const uint16_t *)src,
                           (uint16_t *)dst, W, n_mats, op);
    return check_launch("permute_kernel");
}

template <typename T>
__global__ void zero_padding_kernel(T *__restrict__ packed, int W, int n_mats, int one_padded_in, int unpadded_out) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= W * W) return;
    const int i = idx / W, j = idx % W;
    if (i >= one_padded_in) packed[packed_coord(i, j, W)] = (T)0;
    if (j >= unpadded_out) packed[(size_t)(n_mats - 1) * W * W + packed_coord(i, j, W)] = (T)0;
}

template <typename T>
__global__ void l2_loss_kernel(const T *__restrict__ pred, const float *__restrict__ target, size_t n, float inv_n,
                               float loss_scale, float *__restrict__ values, T *__restrict__ grads) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float diff = (float)pred[i] - target[i];
    if (values) values[i] = diff * diff * inv_n;
    grads[i] = (T)as_fp32(loss_scale * 2 * diff * inv_n);
}

template <typename G, typename P>
__global__ void adam_kernel(float *__restrict__ param, float *__restrict__ m, float *__restrict__ v, const G *__restrict__ grad,
                            float grad_scale, size_t n, float step_size, float bc2_sqrt, float beta1, float beta2, float eps,
                            P *__restrict__ param_T) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float g = (float)grad[i] * grad_scale;
    const float mi = m[i] + (1.0f - beta1) * (g - m[i]);
    const float vi = beta2 * v[i] + (1.0f - beta2) * g * g;
    m[i] = mi;
    v[i] = vi;
    const float denom = sqrtf(vi) / bc2_sqrt + eps;
    const float p = param[i] - step_size * (mi / denom);
    param[i] = p;
    if (param_T) param_T[i] = (P)p;
}

template <typename T> __global__ void fill_kernel(T *__restrict__ p, size_t n, T v) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

// Element i := lo + (hi - lo) * u_i, where u_i in [0, 1) is the top 24 bits of the splitmix64 output for the state
// seed + (first + i + 1) * 0x9E3779B97F4A7C15: the value depends on (seed, first + i) only, not on the launch shape.
template <typename T> __global__ void fill_uniform_kernel(T *__restrict__ p, size_t n, float lo, float hi, unsigned long long seed, unsigned long long first) {
    const float span = hi - lo;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        unsigned long long z = seed + (first + i + 1ull) * 0x9E3779B97F4A7C15ull;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        const float u = (float)(unsigned int)(z >> 40) * 5.9604644775390625e-8f; // 2^-24: exact
        p[i] = (T)as_fp32(lo + as_fp32(span * u));
    }
}

template <typename D, typename S> __global__ void cast_kernel(D *__restrict__ d, const S *__restrict__ s, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) d[i] = (D)(float)s[i];
}

// One thread per weight: reads the raw gradient element dW[l][n][k], updates the fp32 master copy (packed
// layout) with Adam, and writes the rounded weight to the packed T copy and to both operand-order copies.
template <typename T>
__global__ void __launch_bounds__(256) mlp_adam_update_kernel(const AdamArgs a, const float *__restrict__ dW_raw, int total) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < total) adam_update_element<T>(a, idx, dW_raw[idx]);
}

} // namespace tnn

using namespace tnn;

TNN_API const char *tnn_last_error(void) { return error_buffer(); }
TNN_API int tnn_abi_version(void) { return TNN_HIP_ABI_VERSION; }

TNN_API int tnn_device_check(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return fail(TNN_ERR_HIP, "hipGetDeviceCount failed");
    }
    int good = 0;
    for (int d = 0; d < n; ++d) {
        hipDeviceProp_t p;
        if (hipGetDeviceProperties(&p, d) == hipSuccess && strncmp(p.gcnArchName, "gfx950", 6) == 0) ++good;
    }
    if (good == 0) return fail(TNN_ERR_HIP, "no gfx950 device among %d HIP devices", n);
    return good;
}

TNN_API int tnn_pack_weights(int dtype, int width, int n_mats, const void *d_unpacked, void *d_packed, tnn_stream_t stream) {
    return launch_permute(dtype, width, n_mats, d_unpacked, d_packed, OP_PACK, as_stream(stream));
}
TNN_API int tnn_unpack_weights(int dtype, int width, int n_mats, const void *d_packed, void *d_unpacked, tnn_stream_t stream) {
    return launch_permute(dtype, width, n_mats, d_packed, d_unpacked, OP_UNPACK, as_stream(stream));
}
TNN_API int tnn_packed_transpose(int dtype, int width, int n_mats, const void *d_packed, void *d_packed_T, tnn_stream_t stream) {
    return launch_permute(dtype, width, n_mats, d_packed, d_packed_T, OP_PACKED_TRANSPOSE, as_stream(stream));
}
TNN_API int tnn_pack_and_transpose(int dtype, int width, int n_mats, const void *d_raw, void *d_packed, tnn_stream_t stream) {
    return launch_permute(dtype, width, n_mats, d_raw, d_packed, OP_PACK_AND_TRANSPOSE, as_stream(stream));
}

TNN_API int tnn_zero_weights_padding(const tnn_mlp_desc *desc, void *d_packed, int unpadded_input_width,
                                     int unpadded_output_width, int use_bias, tnn_stream_t stream) {
    int rc = check_mlp_desc(desc);
    if (rc) return rc;
    if (!d_packed) return fail(TNN_ERR_INVALID_ARGUMENT, "d_packed is NULL");
    const int W = desc->width;
    // include/network/Network.h:172-173
    if (unpadded_input_width > W || unpadded_output_width > W || unpadded_input_width <= 0 || unpadded_output_width <= 0)
        return fail(TNN_ERR_INVALID_ARGUMENT, "Padded weights width cannot be less than the unpadded.");
    // include/network/Network.h:191-202
    int one_padded;
    if (!use_bias)
        one_padded = unpadded_input_width;
    else if (unpadded_input_width % 16 == 0)
        one_padded = W;
    else
        one_padded = (unpadded_input_width / 16 + 1) * 16;
    if (one_padded > W) return fail(TNN_ERR_INVALID_ARGUMENT, "one_padded_input_width > padded_input_width, the input width is too small.");
    const int n_mats = desc->n_hidden_layers + 1;
    TNN_LAUNCH((zero_padding_kernel<uint16_t>), dim3((W * W + 255) / 256), dim3(256), 0, as_stream(stream),
                       (uint16_t *)d_packed, W, n_mats, one_padded, unpadded_output_width);
    return check_launch("zero_padding_kernel");
}

TNN_API int tnn_l2_loss(int dtype, const void *d_predictions, const float *d_targets, size_t n_elements, float loss_scale,
                        float *d_values, void *d_grads, tnn_stream_t stream) {
    if (dtype != TNN_BF16 && dtype != TNN_FP16) return fail(TNN_ERR_UNSUPPORTED, "dtype %d", dtype);
    if (!d_predictions || !d_targets || !d_grads) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (n_elements == 0) return fail(TNN_ERR_INVALID_ARGUMENT, "n_elements == 0");
    // include/losses/loss.h:27-42 rejects a zero loss scale
    if (loss_scale == 0.0f) return fail(TNN_ERR_INVALID_ARGUMENT, "loss_scale must not be 0");
    const float inv_n = 1.0f / (float)n_elements;
    const unsigned blocks = (unsigned)((n_elements + 255) / 256);
    if (dtype == TNN_BF16)
        TNN_LAUNCH((l2_loss_kernel<bf16_t>), dim3(blocks), dim3(256), 0, as_stream(stream), (const bf16_t *)d_predictions,
                           d_targets, n_elements, inv_n, loss_scale, d_values, (bf16_t *)d_grads);
    else
        TNN_LAUNCH((l2_loss_kernel<fp16_t>), dim3(blocks), dim3(256), 0, as_stream(stream), (const fp16_t *)d_predictions,
                           d_targets, n_elements, inv_n, loss_scale, d_values, (fp16_t *)d_grads);
    return check_launch("l2_loss_kernel");
}

template <typename G>
static int launch_adam(float *p, float *m, float *v, const void *g, float gs, size_t n, float step_size, float bc2_sqrt,
                       float b1, float b2, float eps, void *pT, int pT_dtype, hipStream_t s) {
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (pT && pT_dtype == TNN_BF16)
        TNN_LAUNCH((adam_kernel<G, bf16_t>), dim3(blocks), dim3(256), 0, s, p, m, v, (const G *)g, gs, n, step_size,
                           bc2_sqrt, b1, b2, eps, (bf16_t *)pT);
    else if (pT && pT_dtype == TNN_FP16)
        TNN_LAUNCH((adam_kernel<G, fp16_t>), dim3(blocks), dim3(256), 0, s, p, m, v, (const G *)g, gs, n, step_size,
                           bc2_sqrt, b1, b2, eps, (fp16_t *)pT);
    else
        TNN_LAUNCH((adam_kernel<G, float>), dim3(blocks), dim3(256), 0, s, p, m, v, (const G *)g, gs, n, step_size,
                           bc2_sqrt, b1, b2, eps, (float *)pT);
    return check_launch("adam_kernel");
}

TNN_API int tnn_adam_step(float *d_param, float *d_m, float *d_v, const void *d_grad, int grad_dtype, float grad_scale,
                          size_t n, int step, float lr, float beta1, float beta2, float eps, void *d_param_T,
                          int param_T_dtype, tnn_stream_t stream) {
    if (!d_param || !d_m || !d_v || !d_grad) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (step < 1) return fail(TNN_ERR_INVALID_ARGUMENT, "step counts from 1");
    if (n == 0) return TNN_OK;
    if (d_param_T && param_T_dtype != TNN_BF16 && param_T_dtype != TNN_FP16 && param_T_dtype != TNN_FP32)
        return fail(TNN_ERR_UNSUPPORTED, "param_T_dtype %d", param_T_dtype);
    const double bc1 = 1.0 - pow((double)beta1, step);
    const double bc2 = 1.0 - pow((double)beta2, step);
    const float step_size = (float)(lr / bc1);
    const float bc2_sqrt = (float)sqrt(bc2);
    hipStream_t s = as_stream(stream);
    switch (grad_dtype) {
    case TNN_BF16:
        return launch_adam<bf16_t>(d_param, d_m, d_v, d_grad, grad_scale, n, step_size, bc2_sqrt, beta1, beta2, eps, d_param_T,
                                   param_T_dtype, s);
    case TNN_FP16:
        return launch_adam<fp16_t>(d_param, d_m, d_v, d_grad, grad_scale, n, step_size, bc2_sqrt, beta1, beta2, eps, d_param_T,
                                   param_T_dtype, s);
    case TNN_FP32:
        return launch_adam<float>(d_param, d_m, d_v, d_grad, grad_scale, n, step_size, bc2_sqrt, beta1, beta2, eps, d_param_T,
                                  param_T_dtype, s);
    default: return fail(TNN_ERR_UNSUPPORTED, "grad_dtype %d", grad_dtype);
    }
}

TNN_API int tnn_mlp_adam_update(const tnn_mlp_desc *desc, float *d_master_packed, float *d_m, float *d_v, const float *d_dW_raw,
                                float grad_scale, int step, float lr, float beta1, float beta2, float eps, void *d_packed_T,
                                void *d_prepared_fwd, void *d_prepared_bwd, tnn_stream_t stream) {
    int rc = check_mlp_desc(desc);
    if (rc) return rc;
    if (!d_master_packed || !d_m || !d_v || !d_dW_raw) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (step < 1) return fail(TNN_ERR_INVALID_ARGUMENT, "step counts from 1");
    const int W = desc->width, n_mats = desc->n_hidden_layers + 1;
    const int total = W * W * n_mats;
    const AdamArgs a = make_adam_args(d_master_packed, d_m, d_v, grad_scale, step, lr, beta1, beta2, eps, d_packed_T, d_prepared_fwd,
                                      d_prepared_bwd, W);
    hipStream_t s = as_stream(stream);
    if (desc->dtype == TNN_BF16)
        TNN_LAUNCH((mlp_adam_update_kernel<bf16_t>), dim3((total + 255) / 256), dim3(256), 0, s, a, d_dW_raw, total);
    else
        TNN_LAUNCH((mlp_adam_update_kernel<fp16_t>), dim3((total + 255) / 256), dim3(256), 0, s, a, d_dW_raw, total);
    return check_launch("mlp_adam_update_kernel");
}

TNN_API int tnn_fill(int dtype, void *d_ptr, size_t n, float value, tnn_stream_t stream) {
    if (!d_ptr && n) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (n == 0) return TNN_OK;
    size_t blocks = (n + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipStream_t s = as_stream(stream);
    switch (dtype) {
    case TNN_BF16: TNN_LAUNCH((fill_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, s, (bf16_t *)d_ptr, n, (bf16_t)value); break;
    case TNN_FP16: TNN_LAUNCH((fill_kernel<fp16_t>), dim3((unsigned)blocks), dim3(256), 0, s, (fp16_t *)d_ptr, n, (fp16_t)value); break;
    case TNN_FP32: TNN_LAUNCH((fill_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, s, (float *)d_ptr, n, value); break;
    default: return fail(TNN_ERR_UNSUPPORTED, "dtype %d", dtype);
    }
    return check_launch("fill_kernel");
}

TNN_API int tnn_fill_uniform(int dtype, void *d_ptr, size_t n, float lo, float hi, uint64_t seed, uint64_t first_index, tnn_stream_t stream) {
    if (!d_ptr && n) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (!(lo <= hi)) return fail(TNN_ERR_INVALID_ARGUMENT, "tnn_fill_uniform: bounds %g, %g", (double)lo, (double)hi);
    if (n == 0) return TNN_OK;
    size_t blocks = (n + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipStream_t s = as_stream(stream);
    const unsigned long long sd = seed, fi = first_index;
    switch (dtype) {
    case TNN_BF16: TNN_LAUNCH((fill_uniform_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, s, (bf16_t *)d_ptr, n, lo, hi, sd, fi); break;
    case TNN_FP16: TNN_LAUNCH((fill_uniform_kernel<fp16_t>), dim3((unsigned)blocks), dim3(256), 0, s, (fp16_t *)d_ptr, n, lo, hi, sd, fi); break;
    case TNN_FP32: TNN_LAUNCH((fill_uniform_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, s, (float *)d_ptr, n, lo, hi, sd, fi); break;
    default: return fail(TNN_ERR_UNSUPPORTED, "dtype %d", dtype);
    }
    return check_launch("fill_uniform_kernel");
}

template <typename D> static int launch_cast(D *d, int src_dtype, const void *src, size_t n, hipStream_t s) {
    size_t blocks = (n + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    switch (src_dtype) {
    case TNN_BF16: TNN_LAUNCH((cast_kernel<D, bf16_t>), dim3((unsigned)blocks), dim3(256), 0, s, d, (const bf16_t *)src, n); break;
    case TNN_FP16: TNN_LAUNCH((cast_kernel<D, fp16_t>), dim3((unsigned)blocks), dim3(256), 0, s, d, (const fp16_t *)src, n); break;
    case TNN_FP32: TNN_LAUNCH((cast_kernel<D, float>), dim3((unsigned)blocks), dim3(256), 0, s, d, (const float *)src, n); break;
    default: return fail(TNN_ERR_UNSUPPORTED, "src dtype %d", src_dtype);
    }
    return check_launch("cast_kernel");
}

TNN_API int tnn_cast(int dst_dtype, void *d_dst, int src_dtype, const void *d_src, size_t n, tnn_stream_t stream) {
    if ((!d_dst || !d_src) && n) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (n == 0) return TNN_OK;
    hipStream_t s = as_stream(stream);
    switch (dst_dtype) {
    case TNN_BF16: return launch_cast<bf16_t>((bf16_t *)d_dst, src_dtype, d_src, n, s);
    case TNN_FP16: return launch_cast<fp16_t>((fp16_t *)d_dst, src_dtype, d_src, n, s);
    case TNN_FP32: return launch_cast<float>((float *)d_dst, src_dtype, d_src, n, s);
    default: return fail(TNN_ERR_UNSUPPORTED, "dst dtype %d", dst_dtype);
    }
}
