/*
 * tnn_oracle.c -- CPU restatement of the reference algorithms on the hot path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is the checker for the HIP kernels: only
 * the test suite, the smoke check and the cpu_baseline leg of the benchmark may
 * load it. Nothing in the shipped library calls it and it is never a fallback.
 *
 * Every function cites the reference source (paths relative to the reference
 * checkout) whose arithmetic it follows. Plain C99 + OpenMP over batch rows.
 *
 * Pinning status (what independent evidence each function is checked against in
 * tests/test_oracle_*.py):
 *   packing / transposes ........ golden vectors of test/doctest_packing.cpp:21-46,
 *                                 test/doctest_common.cpp:25-119, test/python/test_packing.py:9-48
 *   mlp_forward_f64 ............. closed forms of test/doctest_swiftnet.cpp:44-51,79-96 and
 *                                 benchmarks/benchmark_inference.h:47-48; torch fp64 linear chain
 *   mlp_backward_f64 ............ closed form dW==1 (benchmarks/benchmark_training.h:48-59,90-96);
 *                                 torch fp64 autograd; finite differences
 *   mlp_forward_T / backward_T .. bounded distance to the f64 functions + exactness on
 *                                 inputs where no rounding occurs
 *   l2_loss ..................... closed form of test/doctest_losses.cpp:46-51
 *   adam_step ................... torch.optim.Adam on CPU
 *   grid_* ...................... golden vector test/doctest_encodings.cpp:234-285, zero-gradient
 *                                 case :286-341, brute-force dense indexing, adjoint identity
 *   identity / frequency ........ closed forms of test/doctest_encodings.cpp:156-195,486-584
 *   sh_forward .................. golden rows of test/python/test_encodings.py:389-573 (degree 4), the degree-1 vector of
 *                                 test/doctest_encodings.cpp:197-232, the reference's explicit expressions of bands 0-3
 *                                 (sh_explicit16) and of single members of bands 4-7, orthonormality on the sphere
 *   fill_uniform ................ the library's own seeded generator (no counterpart sequence in the reference): the
 *                                 published splitmix64 test vector, range, mean and variance of the uniform law
 *   default table init / Xavier init of the reference: parity unpinned (unseeded / closed-source
 *   generators in the reference); their sequences are not restated here, only the distribution is matched.
 */
#include <math.h>
#ifndef M_PI
#define M_PI 3.14159265358979323846 /* strict C99 leaves it out of math.h */
#endif
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define TNN_ORACLE_API __attribute__((visibility("default")))

/* Activation codes: order of `enum class Activation` in include/common/common.h:28-38 */
enum { ACT_RELU = 0, ACT_SIGMOID = 4, ACT_NONE = 8 };
/* dtype codes */
enum { DT_BF16 = 0, DT_FP16 = 1, DT_FP32 = 2 };

TNN_ORACLE_API int tnn_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

TNN_ORACLE_API void tnn_oracle_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ------------------------------------------------------------------------- */
/* Rounding to the 2-byte storage types (round-to-nearest-even, denormals kept:
 * include/network/kernel_esimd.h:182-183 runs with denorm_hf_allow).           */
/* ------------------------------------------------------------------------- */
static inline float round_bf16(float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    if ((u & 0x7f800000u) == 0x7f800000u) { /* inf / nan */
        if (u & 0x007fffffu) u |= 0x00400000u;
        u &= 0xffff0000u;
    } else {
        u += 0x7fffu + ((u >> 16) & 1u);
        u &= 0xffff0000u;
    }
    memcpy(&v, &u, 4);
    return v;
}

static inline float round_fp16(float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    const uint32_t sign = u & 0x80000000u;
    uint32_t a = u & 0x7fffffffu;
    float r;
    if (a >= 0x7f800000u) { /* inf / nan */
        r = v;
    } else if (a >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        uint32_t inf = sign | 0x7f800000u;
        memcpy(&r, &inf, 4);
    } else if (a >= 0x38800000u) { /* normal half range: keep 10 mantissa bits */
        a += 0xfffu + ((a >> 13) & 1u);
        a &= 0xffffe000u;
        a |= sign;
        memcpy(&r, &a, 4);
    } else { /* half denormal: quantum 2^-24; adding 1.5*2^-1... trick via float add */
        float av;
        memcpy(&av, &a, 4);
        /* magic = 2^-1: (av + 0.5f) forces rounding at 2^-24 ulp boundary (ulp of [0.5,1) is 2^-24) */
        volatile float t = av + 0.5f;
        av = t - 0.5f;
        memcpy(&a, &av, 4);
        a |= sign;
        memcpy(&r, &a, 4);
    }
    return r;
}

static inline float round_T(float v, int dtype) {
    if (dtype == DT_BF16) return round_bf16(v);
    if (dtype == DT_FP16) return round_fp16(v);
    return v;
}

TNN_ORACLE_API void tnn_oracle_round(const float *in, float *out, size_t n, int dtype) {
    for (size_t i = 0; i < n; ++i) out[i] = round_T(in[i], dtype);
}

/* ------------------------------------------------------------------------- */
/* Packed ("VNNI") weight layout.                                              */
/* ------------------------------------------------------------------------- */

/* source/common/common.cpp:33-42 */
TNN_ORACLE_API unsigned tnn_oracle_to_packed_layout_coord(unsigned idx, unsigned rows, unsigned cols) {
    (void)rows;
    const unsigned i = idx / cols, j = idx % cols;
    return (i % 2 == 0) ? i * cols + 2 * j : (i - 1) * cols + 2 * j + 1;
}

/* source/common/common.cpp:58-66 */
TNN_ORACLE_API unsigned tnn_oracle_from_packed_layout_coord(unsigned idx, unsigned rows, unsigned cols) {
    (void)rows;
    const unsigned i = idx / (cols * 2), j = idx % (cols * 2);
    return (j % 2 == 0) ? (i * 2) * cols + j / 2 : (i * 2 + 1) * cols + (j - 1) / 2;
}

/* include/common/common.h:174-212 (vertical_pack + get_packed_weights); every matrix is W x W
 * because input and output widths are padded to the network width (include/network/Network.h:67-68). */
TNN_ORACLE_API void tnn_oracle_pack_weights(const float *unpacked, float *packed, int n_mats, int W) {
    for (int m = 0; m < n_mats; ++m) {
        const float *src = unpacked + (size_t)m * W * W;
        float *dst = packed + (size_t)m * W * W;
        for (int idx = 0; idx < W * W; ++idx) dst[tnn_oracle_to_packed_layout_coord(idx, W, W)] = src[idx];
    }
}

TNN_ORACLE_API void tnn_oracle_unpack_weights(const float *packed, float *unpacked, int n_mats, int W) {
    for (int m = 0; m < n_mats; ++m) {
        const float *src = packed + (size_t)m * W * W;
        float *dst = unpacked + (size_t)m * W * W;
        for (int idx = 0; idx < W * W; ++idx) dst[idx] = src[tnn_oracle_to_packed_layout_coord(idx, W, W)];
    }
}

/* include/common/DeviceMatrix.h:429-444 : packed(W) -> packed(W^T), per matrix (rows x cols) */
TNN_ORACLE_API void tnn_oracle_packed_transpose(const float *src, float *dst, int rows, int cols) {
    for (int idx = 0; idx < rows * cols; ++idx) {
        const int i = idx / cols, j = idx % cols;
        const int transposed_idx = j * rows + i;
        dst[tnn_oracle_to_packed_layout_coord(idx, cols, rows)] =
            src[tnn_oracle_to_packed_layout_coord(transposed_idx, rows, cols)];
    }
}

/* include/common/DeviceMatrix.h:469-488 : raw [rows][cols] -> transposed, then packed */
TNN_ORACLE_API void tnn_oracle_pack_and_transpose(const float *src, float *dst, int rows, int cols) {
    for (int idx = 0; idx < rows * cols; ++idx) {
        const int i = idx / cols, j = idx % cols;
        const int transposed_idx = j * rows + i;
        dst[tnn_oracle_to_packed_layout_coord(idx, rows, cols)] = src[transposed_idx];
    }
}

/* include/network/Network.h:171-233 : zero rows >= one-padded input width of matrix 0 and
 * columns >= output width of the last matrix. `packed` holds n_mats W x W matrices. */
TNN_ORACLE_API int tnn_oracle_zero_weights_padding(float *packed, int n_mats, int W, int unpadded_in,
                                                   int unpadded_out, int use_bias) {
    if (unpadded_in > W || unpadded_out > W) return -1;
    int one_padded;
    if (!use_bias)
        one_padded = unpadded_in;
    else if (unpadded_in % 16 == 0)
        one_padded = W;
    else
        one_padded = (unpadded_in / 16 + 1) * 16;
    if (one_padded > W) return -1;
    if (one_padded != W) {
        float *w0 = packed;
        for (int idx = 0; idx < W * W; ++idx)
            if (idx / W >= one_padded) w0[tnn_oracle_to_packed_layout_coord(idx, W, W)] = 0.0f;
    }
    if (unpadded_out != W) {
        float *wl = packed + (size_t)(n_mats - 1) * W * W;
        for (int idx = 0; idx < W * W; ++idx)
            if (idx % W >= unpadded_out) wl[tnn_oracle_to_packed_layout_coord(idx, W, W)] = 0.0f;
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* MLP in double precision without intermediate rounding: test/mlp.h.          */
/* Weights are the "unpacked" vector of test/mlp.h:391-402: n_mats matrices,    */
/* element (k=in, n=out) at k*W + n; y[n] = sum_k x[k] * w[k][n].               */
/* ------------------------------------------------------------------------- */
static inline double act_f64(double v, int act) {
    if (act == ACT_RELU) return v > 0.0 ? v : 0.0; /* test/mlp.h:134 */
    if (act == ACT_SIGMOID) return 1.0 / (1.0 + exp(-v)); /* test/mlp.h:143 */
    return v;
}
static inline double dact_f64(double activated, int act) {
    if (act == ACT_RELU) return activated > 0.0 ? 1.0 : 0.0; /* test/mlp.h:140 */
    if (act == ACT_SIGMOID) return activated * (1.0 - activated); /* test/mlp.h:145-149 */
    return 1.0;
}

/* test/mlp.h:234-282. layer_outputs: (n_mats+1) matrices M x W, [0] = copy of x. */
TNN_ORACLE_API void tnn_oracle_mlp_forward_f64(int W, int n_mats, int act, int out_act, const double *w,
                                               const double *x, size_t M, double *layer_outputs) {
    memcpy(layer_outputs, x, M * W * sizeof(double));
#pragma omp parallel for schedule(static)
    for (long long m = 0; m < (long long)M; ++m) {
        for (int l = 0; l < n_mats; ++l) {
            const double *in = layer_outputs + ((size_t)l * M + m) * W;
            double *out = layer_outputs + ((size_t)(l + 1) * M + m) * W;
            const double *wl = w + (size_t)l * W * W;
            const int a = (l == n_mats - 1) ? out_act : act;
            for (int n = 0; n < W; ++n) {
                double s = 0.0;
                for (int k = 0; k < W; ++k) s += wl[k * W + n] * in[k];
                out[n] = act_f64(s, a);
            }
        }
    }
}

/* test/mlp.h:285-389, for a batch and an arbitrary dL/dy (the reference derives dL/dy from an L2
 * loss first, :301-310; that part is tnn_oracle_l2_loss).
 *   deltas: n_mats matrices M x W, deltas[l] = gradient w.r.t. the pre-activation output of matrix l
 *   dW:     n_mats matrices [n=out][k=in] (test/mlp.h:356-368 transposes to [out][in]), summed over rows
 *   dX:     M x W (may be NULL)                                                                   */
TNN_ORACLE_API void tnn_oracle_mlp_backward_f64(int W, int n_mats, int act, int out_act, const double *w,
                                                const double *layer_outputs, const double *dLdy, size_t M,
                                                double *deltas, double *dW, double *dX) {
#pragma omp parallel for schedule(static)
    for (long long m = 0; m < (long long)M; ++m) {
        /* output layer: test/mlp.h:318-329 */
        {
            const double *y = layer_outputs + ((size_t)n_mats * M + m) * W;
            double *d = deltas + ((size_t)(n_mats - 1) * M + m) * W;
            for (int n = 0; n < W; ++n) d[n] = dLdy[m * W + n] * dact_f64(y[n], out_act);
        }
        /* hidden layers: test/mlp.h:332-352 */
        for (int l = n_mats - 2; l >= 0; --l) {
            const double *dn = deltas + ((size_t)(l + 1) * M + m) * W;
            double *d = deltas + ((size_t)l * M + m) * W;
            const double *wl = w + (size_t)(l + 1) * W * W;
            const double *a = layer_outputs + ((size_t)(l + 1) * M + m) * W;
            for (int k = 0; k < W; ++k) {
                double s = 0.0;
                for (int n = 0; n < W; ++n) s += dn[n] * wl[k * W + n];
                d[k] = s * dact_f64(a[k], act);
            }
        }
        if (dX) { /* test/mlp.h:375-388 */
            const double *d0 = deltas + (size_t)m * W;
            for (int k = 0; k < W; ++k) {
                double s = 0.0;
                for (int n = 0; n < W; ++n) s += d0[n] * w[k * W + n];
                dX[m * W + k] = s;
            }
        }
    }
    /* weight gradients: test/mlp.h:362-372, summed over the batch */
#pragma omp parallel for schedule(static) collapse(2)
    for (int l = 0; l < n_mats; ++l) {
        for (int n = 0; n < W; ++n) {
            double *row = dW + ((size_t)l * W + n) * W;
            for (int k = 0; k < W; ++k) row[k] = 0.0;
            for (size_t m = 0; m < M; ++m) {
                const double dv = deltas[((size_t)l * M + m) * W + n];
                if (dv == 0.0) continue;
                const double *a = layer_outputs + ((size_t)l * M + m) * W;
                for (int k = 0; k < W; ++k) row[k] += dv * a[k];
            }
        }
    }
}

/* ------------------------------------------------------------------------- */
/* MLP with the device kernels' rounding points: include/network/kernel_esimd.h */
/* All arrays are float and hold values representable in the storage type T.    */
/* ------------------------------------------------------------------------- */

/* include/network/kernel_esimd.h:443-458 (applyActivation): fp32 accumulator -> T */
static inline float act_T(float acc, int act, int dtype) {
    if (act == ACT_RELU) {
        const float t = round_T(acc, dtype);
        return t > 0.0f ? t : 0.0f;
    }
    if (act == ACT_SIGMOID) return round_T(1.0f / (1.0f + expf(-acc)), dtype);
    return round_T(acc, dtype);
}

/* include/network/kernel_esimd.h:565-640 (forward_impl_general) with MAD :323-441 (fp32 accumulate).
 * store_interm != 0: interm = (n_mats+1) matrices M x W, [0] = x (training forward, :601-605,620-631)
 * store_interm == 0: interm = 1 matrix M x W holding the network output (inference, :633-635)      */
TNN_ORACLE_API void tnn_oracle_mlp_forward_T(int dtype, int W, int n_mats, int act, int out_act, const float *w,
                                             const float *x, size_t M, float *interm, int store_interm) {
#pragma omp parallel for schedule(static)
    for (long long m = 0; m < (long long)M; ++m) {
        float cur[128], nxt[128];
        for (int k = 0; k < W; ++k) cur[k] = x[m * W + k];
        if (store_interm) memcpy(interm + (size_t)m * W, cur, W * sizeof(float));
        for (int l = 0; l < n_mats; ++l) {
            const float *wl = w + (size_t)l * W * W;
            const int a = (l == n_mats - 1) ? out_act : act;
            float acc[128];
            for (int n = 0; n < W; ++n) acc[n] = 0.0f;
            for (int k = 0; k < W; ++k) {
                const float xv = cur[k];
                const float *wr = wl + (size_t)k * W;
                for (int n = 0; n < W; ++n) acc[n] += xv * wr[n];
            }
            for (int n = 0; n < W; ++n) nxt[n] = act_T(acc[n], a, dtype);
            memcpy(cur, nxt, W * sizeof(float));
            if (store_interm) memcpy(interm + ((size_t)(l + 1) * M + m) * W, cur, W * sizeof(float));
        }
        if (!store_interm) memcpy(interm + (size_t)m * W, cur, W * sizeof(float));
    }
}

/* include/network/kernel_esimd.h:460-487 (applyBackwardActivation) on an fp32 accumulator */
static inline float bwd_act_T(float acc, float fwd, int act, int dtype) {
    if (act == ACT_RELU) return round_T(fwd <= 0.0f ? 0.0f : acc, dtype);
    if (act == ACT_SIGMOID) return round_T(acc * (fwd * (1.0f - fwd)), dtype);
    return round_T(acc, dtype);
}

/* include/network/kernel_esimd.h:160-240 (backward_impl): fused delta propagation (:186-227)
 * followed by the batched dW = delta^T * a product (:230-239).
 *   interm_fwd: (n_mats+1) x M x W as written by the training forward
 *   interm_bwd: n_mats x M x W, [l] = delta_l (:203-216)
 *   dW: n_mats x [n=out][k=in]; accumulated in double, rounded to T when round_dw != 0
 *   dX: optional M x W (:217-226)                                                          */
TNN_ORACLE_API void tnn_oracle_mlp_backward_T(int dtype, int W, int n_mats, int act, int out_act, const float *w,
                                              const float *interm_fwd, const float *dLdy, size_t M,
                                              float *interm_bwd, float *dW, float *dX, int round_dw) {
#pragma omp parallel for schedule(static)
    for (long long m = 0; m < (long long)M; ++m) {
        float cur[128], nxt[128];
        {
            const float *y = interm_fwd + ((size_t)n_mats * M + m) * W;
            for (int n = 0; n < W; ++n) {
                const float g = dLdy[m * W + n];
                /* :193-201 : output activation derivative applied on the loaded T tile */
                cur[n] = (out_act == ACT_NONE) ? g : bwd_act_T(g, y[n], out_act, dtype);
            }
            memcpy(interm_bwd + ((size_t)(n_mats - 1) * M + m) * W, cur, W * sizeof(float));
        }
        for (int l = n_mats - 1; l > 0; --l) {
            const float *wl = w + (size_t)l * W * W;
            const float *f = interm_fwd + ((size_t)l * M + m) * W;
            for (int k = 0; k < W; ++k) {
                float acc = 0.0f;
                const float *wr = wl + (size_t)k * W;
                for (int n = 0; n < W; ++n) acc += cur[n] * wr[n];
                nxt[k] = bwd_act_T(acc, f[k], act, dtype);
            }
            memcpy(cur, nxt, W * sizeof(float));
            memcpy(interm_bwd + ((size_t)(l - 1) * M + m) * W, cur, W * sizeof(float));
        }
        if (dX) {
            for (int k = 0; k < W; ++k) {
                float acc = 0.0f;
                const float *wr = w + (size_t)k * W;
                for (int n = 0; n < W; ++n) acc += cur[n] * wr[n];
                dX[m * W + k] = round_T(acc, dtype);
            }
        }
    }
#pragma omp parallel for schedule(static) collapse(2)
    for (int l = 0; l < n_mats; ++l) {
        for (int n = 0; n < W; ++n) {
            double row[128];
            for (int k = 0; k < W; ++k) row[k] = 0.0;
            for (size_t m = 0; m < M; ++m) {
                const double dv = interm_bwd[((size_t)l * M + m) * W + n];
                if (dv == 0.0) continue;
                const float *a = interm_fwd + ((size_t)l * M + m) * W;
                for (int k = 0; k < W; ++k) row[k] += dv * (double)a[k];
            }
            float *o = dW + ((size_t)l * W + n) * W;
            for (int k = 0; k < W; ++k) o[k] = round_dw ? round_T((float)row[k], dtype) : (float)row[k];
        }
    }
}

/* include/losses/l2.h:19-40 : value = (p-t)^2/N, grad = T(loss_scale*2*(p-t)/N), N = all elements */
TNN_ORACLE_API void tnn_oracle_l2_loss(int dtype, const float *pred, const float *target, size_t n_elements,
                                       float loss_scale, float *values, float *grads) {
    const float inv_n = 1.0f / (float)n_elements;
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)n_elements; ++i) {
        const float diff = pred[i] - target[i];
        values[i] = diff * diff * inv_n;
        grads[i] = round_T(loss_scale * 2 * diff * inv_n, dtype);
    }
}

/* Adam as used by the reference's training loops: torch.optim.Adam on the fp32 parameter
 * (dpcpp_bindings/tiny_dpcpp_nn/modules.py:171-175, test/python/test_compare_torch_dpcpp.py:37).
 * Textbook recurrences with bias correction, no weight decay, no amsgrad; step counts from 1. */
TNN_ORACLE_API void tnn_oracle_adam_step(float *param, float *m, float *v, const float *grad, size_t n, int step,
                                         float lr, float beta1, float beta2, float eps) {
    const double bc1 = 1.0 - pow((double)beta1, step);
    const double bc2 = 1.0 - pow((double)beta2, step);
    const float step_size = (float)(lr / bc1);
    const float bc2_sqrt = (float)sqrt(bc2);
    for (size_t i = 0; i < n; ++i) {
        const float g = grad[i];
        m[i] = m[i] + (1.0f - beta1) * (g - m[i]);
        v[i] = beta2 * v[i] + (1.0f - beta2) * g * g;
        const float denom = sqrtf(v[i]) / bc2_sqrt + eps;
        param[i] -= step_size * (m[i] / denom);
    }
}

/* ------------------------------------------------------------------------- */
/* Multi-resolution hash grid.                                                 */
/* ------------------------------------------------------------------------- */
#define GRID_MAX_LEVELS 128 /* include/encodings/grid_interface.h:23 */
enum { GRID_HASH = 0, GRID_DENSE = 1, GRID_TILED = 2 };           /* include/encodings/encoding.h GridType */
enum { HASH_PRIME = 0, HASH_COHERENT_PRIME = 1, HASH_REVERSED_PRIME = 2, HASH_RNG = 3 };
enum { INTERP_NEAREST = 0, INTERP_LINEAR = 1, INTERP_SMOOTHSTEP = 2 };

/* include/common/common_device.h:767-775 */
static inline float grid_scale(uint32_t level, float log2_per_level_scale, uint32_t base_resolution) {
    return exp2f((float)level * log2_per_level_scale) * (float)base_resolution - 1.0f;
}
static inline uint32_t grid_resolution(float scale) { return (uint32_t)ceilf(scale) + 1u; }

static inline uint32_t powi_u32(uint32_t base, uint32_t e) { /* include/common/common.h powi */
    uint32_t r = 1;
    for (uint32_t i = 0; i < e; ++i) r *= base;
    return r;
}

/* include/encodings/grid.h:604-644 : per-level entry counts and prefix-sum offsets (in entries).
 * offsets has n_levels+1 slots; scales/resolutions n_levels. Returns 0, or -1 on bad arguments. */
TNN_ORACLE_API int tnn_oracle_grid_offsets(int n_dims, int n_levels, int log2_hashmap_size, int base_resolution,
                                           float per_level_scale, int grid_type, uint32_t *offsets,
                                           float *scales, uint32_t *resolutions) {
    if (n_levels > GRID_MAX_LEVELS || n_levels <= 0) return -1;
    const float log2_pls = log2f(per_level_scale);
    uint32_t offset = 0;
    for (int i = 0; i < n_levels; ++i) {
        const float scale = grid_scale((uint32_t)i, log2_pls, (uint32_t)base_resolution);
        const uint32_t resolution = grid_resolution(scale);
        const uint32_t max_params = UINT32_MAX / 2;
        uint32_t params_in_level = powf((float)resolution, (float)n_dims) > (float)max_params
                                       ? max_params
                                       : powi_u32(resolution, (uint32_t)n_dims);
        params_in_level = (params_in_level + 7u) / 8u * 8u;
        if (grid_type == GRID_DENSE) {
        } else if (grid_type == GRID_TILED) {
            const uint32_t t = powi_u32((uint32_t)base_resolution, (uint32_t)n_dims);
            if (t < params_in_level) params_in_level = t;
        } else if (grid_type == GRID_HASH) {
            const uint32_t t = 1u << log2_hashmap_size;
            if (t < params_in_level) params_in_level = t;
        } else
            return -1;
        offsets[i] = offset;
        if (scales) scales[i] = scale;
        if (resolutions) resolutions[i] = resolution;
        offset += params_in_level;
    }
    offsets[n_levels] = offset;
    return 0;
}

/* include/common/common_device.h:700-743 */
static inline uint32_t grid_hash(const uint32_t *pos, int n_dims, int hash_type) {
    static const uint32_t prime[7] = {1958374283u, 2654435761u, 805459861u, 3674653429u,
                                      2097192037u, 1434869437u, 2165219737u};
    static const uint32_t coherent[7] = {1u, 2654435761u, 805459861u, 3674653429u,
                                         2097192037u, 1434869437u, 2165219737u};
    static const uint32_t reversed[7] = {2165219737u, 1434869437u, 2097192037u, 3674653429u,
                                         805459861u, 2654435761u, 1958374283u};
    const uint32_t *f;
    if (hash_type == HASH_PRIME)
        f = prime;
    else if (hash_type == HASH_COHERENT_PRIME)
        f = coherent;
    else if (hash_type == HASH_REVERSED_PRIME)
        f = reversed;
    else
        return 0;
    uint32_t r = 0;
    for (int i = 0; i < n_dims; ++i) r ^= pos[i] * f[i];
    return r;
}

/* include/common/common_device.h:745-765 */
static inline uint32_t grid_index(int grid_type, int hash_type, int n_dims, uint32_t hashmap_size,
                                  uint32_t resolution, const uint32_t *pos) {
    uint32_t stride = 1, index = 0;
    for (int dim = 0; dim < n_dims && stride <= hashmap_size; ++dim) {
        index += pos[dim] * stride;
        stride *= resolution;
    }
    if (grid_type == GRID_HASH && hashmap_size < stride) index = grid_hash(pos, n_dims, hash_type);
    return index % hashmap_size;
}

static inline float smoothstep_f(float v) { return v * v * (3.0f - 2.0f * v); } /* common_device.h:787 */

/* Position -> (cell, fractional weight) : include/encodings/grid.h:73-93 */
static inline void grid_cell(int n_dims, int interp, float scale, const float *x, uint32_t *cell, float *frac) {
    for (int d = 0; d < n_dims; ++d) {
        float p = fmaf(scale, x[d], 0.5f);
        const float t = floorf(p);
        cell[d] = (uint32_t)(int)t;
        p -= t;
        frac[d] = (interp == INTERP_SMOOTHSTEP) ? smoothstep_f(p) : p;
    }
}

/* Table index of every (point, level, corner): the bit-exact part of include/encodings/grid.h:95-129.
 * indices: M x n_levels x 2^n_dims (entry index inside the level, before the *F feature stride);
 * cells (optional): M x n_levels x n_dims. */
TNN_ORACLE_API int tnn_oracle_grid_indices(int n_dims, int n_levels, int log2_hashmap_size, int base_resolution,
                                           float per_level_scale, int grid_type, int hash_type, int interp,
                                           const float *x, size_t M, uint32_t *indices, uint32_t *cells) {
    uint32_t offsets[GRID_MAX_LEVELS + 1];
    float scales[GRID_MAX_LEVELS];
    uint32_t res[GRID_MAX_LEVELS];
    if (n_dims > 7 || n_dims < 1) return -1;
    if (tnn_oracle_grid_offsets(n_dims, n_levels, log2_hashmap_size, base_resolution, per_level_scale, grid_type,
                                offsets, scales, res))
        return -1;
    const int nc = 1 << n_dims;
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)M; ++i) {
        for (int l = 0; l < n_levels; ++l) {
            const uint32_t hs = offsets[l + 1] - offsets[l];
            uint32_t cell[7], loc[7];
            float frac[7];
            grid_cell(n_dims, interp, scales[l], x + (size_t)i * n_dims, cell, frac);
            if (cells)
                for (int d = 0; d < n_dims; ++d) cells[((size_t)i * n_levels + l) * n_dims + d] = cell[d];
            for (int c = 0; c < nc; ++c) {
                for (int d = 0; d < n_dims; ++d) loc[d] = (c & (1 << d)) ? cell[d] + 1 : cell[d];
                indices[((size_t)i * n_levels + l) * nc + c] = grid_index(grid_type, hash_type, n_dims, hs, res[l], loc);
            }
        }
    }
    return 0;
}

/* include/encodings/grid.h:37-135 (kernel_grid) + zero padding :682-694.
 * table: flat, (offset[l] + e)*F + f ; out: M x padded_width, column l*F + f. */
TNN_ORACLE_API int tnn_oracle_grid_forward(int n_dims, int n_levels, int F, int log2_hashmap_size,
                                           int base_resolution, float per_level_scale, int grid_type,
                                           int hash_type, int interp, const float *table, const float *x, size_t M,
                                           float *out, int padded_width) {
    uint32_t offsets[GRID_MAX_LEVELS + 1];
    float scales[GRID_MAX_LEVELS];
    uint32_t res[GRID_MAX_LEVELS];
    if (n_dims > 7 || n_dims < 1 || F > 8 || padded_width < n_levels * F) return -1;
    if (tnn_oracle_grid_offsets(n_dims, n_levels, log2_hashmap_size, base_resolution, per_level_scale, grid_type,
                                offsets, scales, res))
        return -1;
    const int nc = 1 << n_dims;
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)M; ++i) {
        float *o = out + (size_t)i * padded_width;
        for (int c = n_levels * F; c < padded_width; ++c) o[c] = 0.0f;
        for (int l = 0; l < n_levels; ++l) {
            const float *g = table + (size_t)offsets[l] * F;
            const uint32_t hs = offsets[l + 1] - offsets[l];
            uint32_t cell[7], loc[7];
            float frac[7], result[8];
            grid_cell(n_dims, interp, scales[l], x + (size_t)i * n_dims, cell, frac);
            if (interp == INTERP_NEAREST) {
                const uint32_t idx = grid_index(grid_type, hash_type, n_dims, hs, res[l], cell) * (uint32_t)F;
                for (int f = 0; f < F; ++f) o[l * F + f] = g[idx + f];
                continue;
            }
            for (int f = 0; f < F; ++f) result[f] = 0.0f;
            for (int c = 0; c < nc; ++c) {
                float weight = 1.0f;
                for (int d = 0; d < n_dims; ++d) {
                    if ((c & (1 << d)) == 0) {
                        weight *= 1 - frac[d];
                        loc[d] = cell[d];
                    } else {
                        weight *= frac[d];
                        loc[d] = cell[d] + 1;
                    }
                }
                const uint32_t idx = grid_index(grid_type, hash_type, n_dims, hs, res[l], loc) * (uint32_t)F;
                for (int f = 0; f < F; ++f) result[f] = fmaf(weight, g[idx + f], result[f]);
            }
            for (int f = 0; f < F; ++f) o[l * F + f] = result[f];
        }
    }
    return 0;
}

/* include/encodings/grid.h:137-245 (kernel_grid_backward), Overwrite mode (:758-762), no stochastic
 * interpolation. The reference adds with relaxed float atomics in arbitrary order; this restatement
 * sums every entry in double and rounds once, i.e. it is the value all orders approximate.
 * grad_table has the shape of the table. */
TNN_ORACLE_API int tnn_oracle_grid_backward(int n_dims, int n_levels, int F, int log2_hashmap_size,
                                            int base_resolution, float per_level_scale, int grid_type,
                                            int hash_type, int interp, const float *x, const float *dLdy, size_t M,
                                            int padded_width, float *grad_table) {
    uint32_t offsets[GRID_MAX_LEVELS + 1];
    float scales[GRID_MAX_LEVELS];
    uint32_t res[GRID_MAX_LEVELS];
    if (n_dims > 7 || n_dims < 1 || F > 8 || padded_width < n_levels * F) return -1;
    if (tnn_oracle_grid_offsets(n_dims, n_levels, log2_hashmap_size, base_resolution, per_level_scale, grid_type,
                                offsets, scales, res))
        return -1;
    const int nc = 1 << n_dims;
    const size_t n_params = (size_t)offsets[n_levels] * F;
    double *acc = (double *)calloc(n_params, sizeof(double));
    if (!acc) return -2;
    /* levels write disjoint table ranges: parallel over levels is race-free */
#pragma omp parallel for schedule(dynamic, 1)
    for (int l = 0; l < n_levels; ++l) {
        double *g = acc + (size_t)offsets[l] * F;
        const uint32_t hs = offsets[l + 1] - offsets[l];
        for (size_t i = 0; i < M; ++i) {
            uint32_t cell[7], loc[7];
            float frac[7];
            grid_cell(n_dims, interp, scales[l], x + i * n_dims, cell, frac);
            const float *gy = dLdy + i * padded_width + l * F;
            if (interp == INTERP_NEAREST) {
                const uint32_t idx = grid_index(grid_type, hash_type, n_dims, hs, res[l], cell) * (uint32_t)F;
                for (int f = 0; f < F; ++f) g[idx + f] += (double)gy[f];
                continue;
            }
            for (int c = 0; c < nc; ++c) {
                float weight = 1.0f;
                for (int d = 0; d < n_dims; ++d) {
                    if ((c & (1 << d)) == 0) {
                        weight *= 1 - frac[d];
                        loc[d] = cell[d];
                    } else {
                        weight *= frac[d];
                        loc[d] = cell[d] + 1;
                    }
                }
                const uint32_t idx = grid_index(grid_type, hash_type, n_dims, hs, res[l], loc) * (uint32_t)F;
                /* grid.h:182 : (GRAD_T)weight * grad[i] is a float product */
                for (int f = 0; f < F; ++f) g[idx + f] += (double)(weight * gy[f]);
            }
        }
    }
    for (size_t p = 0; p < n_params; ++p) grad_table[p] = (float)acc[p];
    free(acc);
    return 0;
}

/* ------------------------------------------------------------------------- */
/* Encodings without parameters                                               */
/* ------------------------------------------------------------------------- */

/* include/encodings/identity.h:61-75 : in * scale + offset, ones beyond the encoded columns */
TNN_ORACLE_API void tnn_oracle_identity_forward(const float *x, int n_dims, float scale, float offset, size_t M, float *out,
                                                int padded_width) {
    for (size_t i = 0; i < M; ++i)
        for (int j = 0; j < padded_width; ++j)
            out[i * padded_width + j] = j >= n_dims ? 1.0f : x[i * n_dims + j] * scale + offset;
}

/* include/encodings/frequency.h:62-86 : the argument is float * size_t (a float product), times M_PI and plus the
 * phase shift in double, rounded to float once; sine in float. dy_dx (may be NULL): M x (n_dims * n_freq * 2). */
TNN_ORACLE_API void tnn_oracle_frequency_forward(const float *x, int n_dims, int n_freq, size_t M, float *out, int padded_width,
                                                 float *dy_dx) {
    const int width = n_dims * n_freq * 2;
    for (size_t i = 0; i < M; ++i)
        for (int j = 0; j < padded_width; ++j) {
            if (j >= width) {
                out[i * padded_width + j] = 1.0f;
                continue;
            }
            const int feature = j / (n_freq * 2), log2_frequency = (j / 2) % n_freq;
            const float phase_shift = (float)((j % 2) * (M_PI / 2.0f));
            const float scaled = x[i * n_dims + feature] * (float)((size_t)1 << log2_frequency);
            const float arg = (float)((double)scaled * M_PI + (double)phase_shift);
            out[i * padded_width + j] = sinf(arg);
            if (dy_dx) dy_dx[i * width + j] = (float)((double)(float)((size_t)1 << log2_frequency) * M_PI * (double)cosf(arg));
        }
}

/* include/encodings/frequency.h:108-126 */
TNN_ORACLE_API void tnn_oracle_frequency_backward(const float *dLdy, int padded_width, const float *dy_dx, int n_dims, int n_freq,
                                                  size_t M, float *dLdx) {
    const int per_input = n_freq * 2, width = n_dims * per_input;
    for (size_t i = 0; i < M; ++i)
        for (int j = 0; j < n_dims; ++j) {
            double r = 0.0;
            for (int k = 0; k < per_input; ++k)
                r += (double)dLdy[i * padded_width + j * per_input + k] * (double)dy_dx[i * width + j * per_input + k];
            dLdx[i * n_dims + j] = (float)r;
        }
}

/* The first 16 real spherical harmonics as the reference spells them out (include/common/common_device.h:47-70; the
 * constants are the closed forms given in its comments). Arguments are the direction itself (no 2x-1 here). */
TNN_ORACLE_API void tnn_oracle_sh_explicit16(double x, double y, double z, double *o) {
    const double sp = sqrt(M_PI);
    const double xy = x * y, xz = x * z, yz = y * z, x2 = x * x, y2 = y * y, z2 = z * z;
    o[0] = 1.0 / (2.0 * sp);
    o[1] = -sqrt(3.0) * y / (2.0 * sp);
    o[2] = sqrt(3.0) * z / (2.0 * sp);
    o[3] = -sqrt(3.0) * x / (2.0 * sp);
    o[4] = sqrt(15.0) * xy / (2.0 * sp);
    o[5] = -sqrt(15.0) * yz / (2.0 * sp);
    o[6] = sqrt(5.0) * (3.0 * z2 - 1.0) / (4.0 * sp);
    o[7] = -sqrt(15.0) * xz / (2.0 * sp);
    o[8] = sqrt(15.0) * (x2 - y2) / (4.0 * sp);
    o[9] = sqrt(70.0) * y * (-3.0 * x2 + y2) / (8.0 * sp);
    o[10] = sqrt(105.0) * xy * z / (2.0 * sp);
    o[11] = sqrt(42.0) * y * (1.0 - 5.0 * z2) / (8.0 * sp);
    o[12] = sqrt(7.0) * z * (5.0 * z2 - 3.0) / (4.0 * sp);
    o[13] = sqrt(42.0) * x * (1.0 - 5.0 * z2) / (8.0 * sp);
    o[14] = sqrt(105.0) * z * (x2 - y2) / (4.0 * sp);
    o[15] = sqrt(70.0) * x * (-x2 + 3.0 * y2) / (8.0 * sp);
}

/* include/encodings/spherical_harmonics.h:55-70 with sh_enc (include/common/common_device.h:33-206). The reference's
 * unrolled expressions were generated from the recurrences of appendix A1 of P.-P. Sloan, "Stupid Spherical Harmonics
 * (SH) Tricks" (common_device.h:43-46); this restates those recurrences, in double:
 *   Y(l, m) = K(l,|m|) * P(l,|m|)(z) * { sqrt2 Re (x+iy)^m | 1 | sqrt2 Im (x+iy)^|m| },  index l^2 + l + m,
 *   P(m,m) = (-1)^m (2m-1)!!,  P(m+1,m) = (2m+1) z P(m,m),  P(l,m) = ((2l-1) z P(l-1,m) - (l+m-1) P(l-2,m)) / (l-m).
 * Input x in [0,1]^3 is mapped to the direction 2x-1; columns beyond degree^2 are ones. */
TNN_ORACLE_API int tnn_oracle_sh_forward(int degree, const float *xin, size_t M, float *out, int padded_width) {
    if (degree < 1 || degree > 8 || padded_width < degree * degree) return -1;
    for (size_t i = 0; i < M; ++i) {
        /* the reference forms 2x-1 in float */
        const double x = (double)(xin[i * 3 + 0] * 2.f - 1.f), y = (double)(xin[i * 3 + 1] * 2.f - 1.f),
                     z = (double)(xin[i * 3 + 2] * 2.f - 1.f);
        float *row = out + i * padded_width;
        double cm = 1.0, sm = 0.0, pmm = 1.0;
        for (int m = 0; m < degree; ++m) {
            if (m > 0) {
                const double cn = cm * x - sm * y;
                sm = cm * y + sm * x;
                cm = cn;
                pmm *= -(double)(2 * m - 1);
            }
            double p2 = 0.0, p1 = pmm;
            for (int l = m; l < degree; ++l) {
                double p;
                if (l == m) {
                    p = pmm;
                } else if (l == m + 1) {
                    p = (2 * m + 1) * z * pmm;
                } else {
                    p = ((2 * l - 1) * z * p1 - (l + m - 1) * p2) / (l - m);
                }
                if (l > m) {
                    p2 = p1;
                    p1 = p;
                }
                double ratio = 1.0;
                for (int t = l - m + 1; t <= l + m; ++t) ratio /= (double)t;
                const double k = sqrt((2.0 * l + 1.0) / (4.0 * M_PI) * ratio) * (m > 0 ? sqrt(2.0) : 1.0);
                if (m == 0) {
                    row[l * l + l] = (float)(k * p);
                } else {
                    row[l * l + l + m] = (float)(k * p * cm);
                    row[l * l + l - m] = (float)(k * p * sm);
                }
            }
        }
        for (int j = degree * degree; j < padded_width; ++j) row[j] = 1.0f;
    }
    return 0;
}

/* The library's seeded uniform fill (tnn_fill_uniform): stands where the reference draws from oneMKL philox
 * (include/common/DeviceMatrix.h:169-178) and from std::mt19937(std::random_device) (include/network/Network.h:271-295).
 * splitmix64 (Steele, Lea, Flood 2014; Vigna's public-domain splitmix64.c): state += gamma per draw, output = mix(state). */
TNN_ORACLE_API uint64_t tnn_oracle_splitmix64(uint64_t seed, uint64_t index) {
    uint64_t z = seed + (index + 1ull) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

TNN_ORACLE_API void tnn_oracle_fill_uniform(float *out, size_t n, float lo, float hi, uint64_t seed, uint64_t first_index, int dtype) {
    const float span = hi - lo;
    for (size_t i = 0; i < n; ++i) {
        const float u = (float)(uint32_t)(tnn_oracle_splitmix64(seed, first_index + i) >> 40) * 5.9604644775390625e-8f;
        const volatile float prod = span * u; /* two roundings, as the kernel */
        out[i] = round_T(lo + prod, dtype);
    }
}
