// Parameter-free input encodings: identity, frequency, spherical harmonics (include/encodings/identity.h,
// frequency.h, spherical_harmonics.h of the reference). Unlike the grid they pad their rows with ones.
// All three are bound by the output write (one row per thread, 16-byte stores where the row allows it).
#include <cmath>

#include "tnn_internal.h"

namespace tnn {

constexpr int kEncThreads = 256;

template <typename O> __device__ __forceinline__ void store_out(O *p, float v) { *p = (O)v; }

// identity.h:61-75: out[i][j] = in[i][j] * scale + offset for j < n_dims, 1 beyond.
template <typename O>
__global__ void __launch_bounds__(kEncThreads)
    identity_kernel(const float *__restrict__ x, O *__restrict__ out, uint32_t n_dims, uint32_t padded, float scale, float offset,
                    size_t n_elements) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n_elements; e += (size_t)gridDim.x * blockDim.x) {
        const size_t i = e / padded;
        const uint32_t j = (uint32_t)(e - i * padded);
        out[e] = (j >= n_dims) ? (O)1.0f : (O)as_fp32(x[i * n_dims + j] * scale + offset);
    }
}

// frequency.h:62-86: column j of a row encodes input feature j / (2 n_f) at frequency 2^((j / 2) % n_f) pi, sine for
// even j and cosine (a phase shift of pi / 2) for odd j. The argument is formed in double and rounded to float once, as
// the reference's expression does (float * size_t * M_PI + phase); dy/dx optionally kept for the backward pass.
template <typename O>
__global__ void __launch_bounds__(kEncThreads)
    frequency_kernel(const float *__restrict__ x, O *__restrict__ out, float *__restrict__ dy_dx, uint32_t n_dims, uint32_t n_freq,
                     uint32_t padded, size_t n_elements) {
    const uint32_t width = n_dims * n_freq * 2;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n_elements; e += (size_t)gridDim.x * blockDim.x) {
        const size_t i = e / padded;
        const uint32_t j = (uint32_t)(e - i * padded);
        if (j >= width) {
            out[e] = (O)1.0f;
            continue;
        }
        const uint32_t feature = j / (n_freq * 2), log2_frequency = (j / 2) % n_freq;
        const float phase_shift = (float)((j % 2) * (M_PI / 2.0f));
        const float pow2 = (float)((size_t)1 << log2_frequency);
        const float arg = (float)((double)(x[i * n_dims + feature] * pow2) * M_PI + (double)phase_shift);
        out[e] = (O)sinf(arg);
        if (dy_dx) dy_dx[i * width + j] = (float)((double)pow2 * M_PI * (double)cosf(arg));
    }
}

// frequency.h:108-126: dL/dx[i][j] = sum_k dL/dy[i][j * 2 n_f + k] * dy/dx[i][j * 2 n_f + k]
template <typename G>
__global__ void __launch_bounds__(kEncThreads)
    frequency_backward_kernel(const G *__restrict__ dLdy, const float *__restrict__ dy_dx, float *__restrict__ dLdx, uint32_t n_dims,
                              uint32_t n_freq, uint32_t padded, size_t n_elements) {
    const uint32_t per_input = n_freq * 2, width = n_dims * per_input;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n_elements; e += (size_t)gridDim.x * blockDim.x) {
        const size_t i = e / n_dims;
        const uint32_t j = (uint32_t)(e - i * n_dims);
        float result = 0.0f;
        for (uint32_t k = 0; k < per_input; ++k)
            result = fmaf((float)dLdy[i * padded + j * per_input + k], dy_dx[i * width + j * per_input + k], result);
        dLdx[e] = result;
    }
}

// Normalisation constants of the real spherical harmonics, K[l][m] = sqrt((2l+1)/(4 pi) (l-m)!/(l+m)!), times sqrt(2) for m > 0.
struct ShConstants {
    float k[8][8];
};

// Real spherical harmonics of bands 0 .. degree-1 at the direction (2x-1, 2y-1, 2z-1), in the polynomial form of Sloan's
// "Stupid Spherical Harmonics Tricks", appendix A1, which the reference's unrolled expressions were generated from
// (include/common/common_device.h:33-206): Y(l, m) = K(l, |m|) * P(l, |m|)(z) * (Re or Im of (x + iy)^|m|), with P the
// associated Legendre function divided by (1 - z^2)^(m/2), a polynomial in z. Output index l^2 + l + m. No unit-length
// assumption is made on the input, exactly as in the reference's expressions.
template <typename O, int DEGREE>
__global__ void __launch_bounds__(kEncThreads)
    sh_kernel(const float *__restrict__ xin, O *__restrict__ out, const ShConstants c, uint32_t padded, size_t M) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= M) return;
    const float x = xin[i * 3 + 0] * 2.f - 1.f, y = xin[i * 3 + 1] * 2.f - 1.f, z = xin[i * 3 + 2] * 2.f - 1.f;
    O *row = out + i * padded;
    float cm = 1.0f, sm = 0.0f; // real and imaginary part of (x + iy)^m
    float pmm = 1.0f;           // P(m, m) = (-1)^m (2m - 1)!!
#pragma unroll
    for (int m = 0; m < DEGREE; ++m) {
        if (m > 0) {
            const float cn = cm * x - sm * y;
            sm = cm * y + sm * x;
            cm = cn;
            pmm *= -(float)(2 * m - 1);
        }
        float p2 = 0.0f, p1 = pmm; // P(l-2, m), P(l-1, m)
#pragma unroll
        for (int l = m; l < DEGREE; ++l) {
            float p;
            if (l == m)
                p = pmm;
            else if (l == m + 1)
                p = (float)(2 * m + 1) * z * pmm;
            else
                p = ((float)(2 * l - 1) * z * p1 - (float)(l + m - 1) * p2) / (float)(l - m);
            if (l > m) {
                p2 = p1;
                p1 = p;
            }
            const float k = c.k[l][m] * p;
            if (m == 0) {
                row[l * l + l] = (O)k;
            } else {
                row[l * l + l + m] = (O)(k * cm);
                row[l * l + l - m] = (O)(k * sm);
            }
        }
    }
    for (uint32_t j = DEGREE * DEGREE; j < padded; ++j) row[j] = (O)1.0f;
}

static unsigned enc_blocks(size_t n) {
    size_t b = (n + kEncThreads - 1) / kEncThreads;
    return (unsigned)(b > 65536 ? 65536 : (b < 1 ? 1 : b));
}

} // namespace tnn

using namespace tnn;

TNN_API int tnn_identity_forward(const float *d_x, uint32_t n_dims, float scale, float offset, void *d_out, int out_dtype,
                                 uint32_t padded_width, size_t M, tnn_stream_t stream) {
    if (n_dims == 0) return fail(TNN_ERR_INVALID_ARGUMENT, "Input width cannot be zero");
    if (padded_width < n_dims) return fail(TNN_ERR_INVALID_ARGUMENT, "Padded output width cannot be less than output width");
    if (M == 0) return TNN_OK;
    if (!d_x || !d_out) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    const size_t n = M * padded_width;
    hipStream_t s = as_stream(stream);
    switch (out_dtype) {
    case TNN_FP32: TNN_LAUNCH((identity_kernel<float>), dim3(enc_blocks(n)), dim3(kEncThreads), 0, s, d_x, (float *)d_out, n_dims, padded_width, scale, offset, n); break;
    case TNN_BF16: TNN_LAUNCH((identity_kernel<bf16_t>), dim3(enc_blocks(n)), dim3(kEncThreads), 0, s, d_x, (bf16_t *)d_out, n_dims, padded_width, scale, offset, n); break;
    case TNN_FP16: TNN_LAUNCH((identity_kernel<fp16_t>), dim3(enc_blocks(n)), dim3(kEncThreads), 0, s, d_x, (fp16_t *)d_out, n_dims, padded_width, scale, offset, n); break;
    default: return fail(TNN_ERR_UNSUPPORTED, "out_dtype %d", out_dtype);
    }
    return check_launch("identity_kernel");
}

static int check_frequency(uint32_t n_dims, uint32_t n_frequencies, uint32_t padded_width) {
    if (n_dims == 0) return fail(TNN_ERR_INVALID_ARGUMENT, "Input width cannot be zero");
    if (n_frequencies == 0) return fail(TNN_ERR_INVALID_ARGUMENT, "Output width cannot be zero");
    if (n_frequencies > 63) return fail(TNN_ERR_INVALID_ARGUMENT, "n_frequencies %u: at most 63", n_frequencies);
    if (0xffffffffu / n_frequencies < 2 * n_dims) return fail(TNN_ERR_INVALID_ARGUMENT, "n_frequencies * 2 * n_dims_to_encode exceeds uint32_t max");
    if (padded_width < n_dims * n_frequencies * 2) return fail(TNN_ERR_INVALID_ARGUMENT, "Padded output width cannot be less than output width");
    return TNN_OK;
}

TNN_API int tnn_frequency_forward(const float *d_x, uint32_t n_dims, uint32_t n_frequencies, void *d_out, int out_dtype,
                                  uint32_t padded_width, float *d_dy_dx, size_t M, tnn_stream_t stream) {
    int rc = check_frequency(n_dims, n_frequencies, padded_width);
    if (rc) return rc;
    if (M == 0) return TNN_OK;
    if (!d_x || !d_out) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    const size_t n = M * padded_width;
    hipStream_t s = as_stream(stream);
    switch (out_dtype) {
    case TNN_FP32: TNN_LAUNCH((frequency_kernel<float>), dim3(enc_blocks(n)), dim3(kEncThreads), 0, s, d_x, (float *)d_out, d_dy_dx, n_dims, n_frequencies, padded_width, n); break;
    case TNN_BF16: TNN_LAUNCH((frequency_kernel<bf16_t>), dim3(enc_blocks(n)), dim3(kEncThreads), 0, s, d_x, (bf16_t *)d_out, d_dy_dx, n_dims, n_frequencies, padded_width, n); break;
    case TNN_FP16: TNN_LAUNCH((frequency_kernel<fp16_t>), dim3(enc_blocks(n)), dim3(kEncThreads), 0, s, d_x, (fp16_t *)d_out, d_dy_dx, n_dims, n_frequencies, padded_width, n); break;
    default: return fail(TNN_ERR_UNSUPPORTED, "out_dtype %d", out_dtype);
    }
    return check_launch("frequency_kernel");
}

TNN_API int tnn_frequency_backward(const void *d_dLdy, int dy_dtype, uint32_t padded_width, const float *d_dy_dx, uint32_t n_dims,
                                   uint32_t n_frequencies, float *d_dLdx, size_t M, tnn_stream_t stream) {
    int rc = check_frequency(n_dims, n_frequencies, padded_width);
    if (rc) return rc;
    if (M == 0) return fail(TNN_ERR_INVALID_ARGUMENT, "batch_size == 0");
    if (!d_dLdy || !d_dy_dx || !d_dLdx) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    const size_t n = M * n_dims;
    hipStream_t s = as_stream(stream);
    switch (dy_dtype) {
    case TNN_FP32: TNN_LAUNCH((frequency_backward_kernel<float>), dim3(enc_blocks(n)), dim3(kEncThreads), 0, s, (const float *)d_dLdy, d_dy_dx, d_dLdx, n_dims, n_frequencies, padded_width, n); break;
    case TNN_BF16: TNN_LAUNCH((frequency_backward_kernel<bf16_t>), dim3(enc_blocks(n)), dim3(kEncThreads), 0, s, (const bf16_t *)d_dLdy, d_dy_dx, d_dLdx, n_dims, n_frequencies, padded_width, n); break;
    case TNN_FP16: TNN_LAUNCH((frequency_backward_kernel<fp16_t>), dim3(enc_blocks(n)), dim3(kEncThreads), 0, s, (const fp16_t *)d_dLdy, d_dy_dx, d_dLdx, n_dims, n_frequencies, padded_width, n); break;
    default: return fail(TNN_ERR_UNSUPPORTED, "dy_dtype %d", dy_dtype);
    }
    return check_launch("frequency_backward_kernel");
}

template <typename O> static int launch_sh(uint32_t degree, const float *x, O *out, const ShConstants &c, uint32_t padded, size_t M, hipStream_t s) {
    const dim3 grid((unsigned)((M + kEncThreads - 1) / kEncThreads)), block(kEncThreads);
    switch (degree) {
    case 1: TNN_LAUNCH((sh_kernel<O, 1>), grid, block, 0, s, x, out, c, padded, M); break;
    case 2: TNN_LAUNCH((sh_kernel<O, 2>), grid, block, 0, s, x, out, c, padded, M); break;
    case 3: TNN_LAUNCH((sh_kernel<O, 3>), grid, block, 0, s, x, out, c, padded, M); break;
    case 4: TNN_LAUNCH((sh_kernel<O, 4>), grid, block, 0, s, x, out, c, padded, M); break;
    case 5: TNN_LAUNCH((sh_kernel<O, 5>), grid, block, 0, s, x, out, c, padded, M); break;
    case 6: TNN_LAUNCH((sh_kernel<O, 6>), grid, block, 0, s, x, out, c, padded, M); break;
    case 7: TNN_LAUNCH((sh_kernel<O, 7>), grid, block, 0, s, x, out, c, padded, M); break;
    default: TNN_LAUNCH((sh_kernel<O, 8>), grid, block, 0, s, x, out, c, padded, M); break;
    }
    return check_launch("sh_kernel");
}

TNN_API int tnn_sh_forward(const float *d_x, uint32_t degree, void *d_out, int out_dtype, uint32_t padded_width, size_t M,
                           tnn_stream_t stream) {
    if (degree == 0 || degree > 8) return fail(TNN_ERR_INVALID_ARGUMENT, "Spherical harmonics degree > 0 and <= 8.");
    if (padded_width < degree * degree) return fail(TNN_ERR_INVALID_ARGUMENT, "Padded output width cannot be less than output width");
    if (M == 0) return TNN_OK;
    if (!d_x || !d_out) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    ShConstants c;
    for (int l = 0; l < 8; ++l)
        for (int m = 0; m < 8; ++m) {
            double k = 0.0;
            if (m <= l) {
                double ratio = 1.0; // (l-m)! / (l+m)!
                for (int t = l - m + 1; t <= l + m; ++t) ratio /= (double)t;
                k = std::sqrt((2.0 * l + 1.0) / (4.0 * M_PI) * ratio) * (m > 0 ? std::sqrt(2.0) : 1.0);
            }
            c.k[l][m] = (float)k;
        }
    hipStream_t s = as_stream(stream);
    switch (out_dtype) {
    case TNN_FP32: return launch_sh<float>(degree, d_x, (float *)d_out, c, padded_width, M, s);
    case TNN_BF16: return launch_sh<bf16_t>(degree, d_x, (bf16_t *)d_out, c, padded_width, M, s);
    case TNN_FP16: return launch_sh<fp16_t>(degree, d_x, (fp16_t *)d_out, c, padded_width, M, s);
    default: return fail(TNN_ERR_UNSUPPORTED, "out_dtype %d", out_dtype);
    }
}
