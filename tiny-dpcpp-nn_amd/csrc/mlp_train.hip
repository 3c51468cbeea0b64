// Fused training step of the MLP for gfx950: forward, L2 loss and its gradient, delta propagation
// and weight gradients in ONE kernel. No activation, delta or loss gradient is written to device
// memory; per workgroup one fp32 partial of every dW and one partial loss leave the chip, and a
// second small kernel sums them in a fixed order.
//
// Reference dataflow being replaced: Trainer::training_step (include/trainer.h:23-46) =
// forward_impl (include/network/kernel_esimd.h:565-640, stores L+2 activation matrices) +
// L2Loss (include/losses/l2.h:19-40) + backward_impl (:160-228, stores L+1 delta matrices) +
// oneMKL gemm_batch (:230-239, re-reads both). Same arithmetic and rounding points.
//
// Per wave: one tile of 32 batch rows; activations of every layer stay in registers (the layer loop
// is unrolled at compile time). Weight gradients contract over batch rows, which live one-per-lane,
// so delta_l and a_l are transposed through LDS: written row-major, read back with the gfx950
// transposing LDS load (ds_read_b64_tr_b16) directly in MFMA operand order.
// Width 64: the four 32x32 tiles of a dW are owned by the four waves of a half-workgroup, which
// share their 4 x 32 rows through LDS. Width <= 32: every wave owns the single tile of its own rows.
#include "mlp_tile.h"

namespace tnn {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

// Two transposing loads = one 8-element MFMA operand. Inside each group of 16 lanes the instruction
// treats the 16 x 8 bytes it reads as a 4 x 16 matrix of 16-bit elements (source lane 4e + q supplies
// row e, columns 4q..4q+3) and hands lane L column L.
template <typename T>
__device__ __forceinline__ typename Storage<T>::vec8 tr_load8(const unsigned char *lds, int off_lo, int off_hi) {
    typedef __attribute__((address_space(3))) s16x4 *lds_ptr;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(lds + off_lo));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(lds + off_hi));
    const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(typename Storage<T>::vec8, v);
}

template <int W> struct TrainShape {
    static constexpr int NK = W / 16;
    static constexpr int NI = (W + 31) / 32;
    static constexpr int GROUP = (NI * NI >= 4) ? 4 : 1; // waves that share rows for one dW
    static constexpr int PITCH = W * 2 + 16;             // bytes per staged row (16-byte skew)
    static constexpr int TILE_BYTES = 32 * PITCH;
    static constexpr int WAVES = kFwdThreads / 64;
    static constexpr int N_GROUPS = WAVES / GROUP;
    static size_t weight_bytes(int n_mats) { return (size_t)n_mats * NI * NK * 64 * 16; }
    static size_t lds_bytes(int n_mats) {
        const size_t stage = (size_t)WAVES * 2 * TILE_BYTES;
        const size_t reduce = (size_t)n_mats * W * W * 4; // end-of-kernel cross-group sum (reuses everything)
        const size_t main = 2 * weight_bytes(n_mats) + stage;
        return main > reduce ? main : reduce;
    }
};

template <typename T, int W, int N_MATS>
__global__ void __launch_bounds__(kFwdThreads)
    mlp_train_fused_kernel(const typename Storage<T>::vec8 *__restrict__ wfwd, const typename Storage<T>::vec8 *__restrict__ wbwd,
                           const T *__restrict__ x, const float *__restrict__ targets, T *__restrict__ y_out,
                           T *__restrict__ dx_out, float *__restrict__ partials, float *__restrict__ loss_partials, int act,
                           int out_act, float loss_scale, float inv_n, long long M) {
    typedef Tile<T, W> TL;
    typedef TrainShape<W> S;
    typedef typename Storage<T>::vec8 vec8;
    constexpr int NK = S::NK, NI = S::NI, GROUP = S::GROUP;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    constexpr int per_mat = NI * NK * kWaveSize; // fragments per matrix
    vec8 *lds_wf = reinterpret_cast<vec8 *>(smem_raw);
    vec8 *lds_wb = lds_wf + N_MATS * per_mat;
    unsigned char *stage = reinterpret_cast<unsigned char *>(lds_wb + N_MATS * per_mat);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 31, h = lane >> 5;

    for (int f = threadIdx.x; f < N_MATS * per_mat; f += kFwdThreads) {
        lds_wf[f] = wfwd[f];
        lds_wb[f] = wbwd[f];
    }
    __syncthreads();

    // staging slots: [wave][0 = delta, 1 = activation][32 rows][PITCH]
    unsigned char *my_d = stage + (size_t)(wave * 2 + 0) * S::TILE_BYTES;
    unsigned char *my_a = stage + (size_t)(wave * 2 + 1) * S::TILE_BYTES;
    const int wr_off = j * S::PITCH + h * 16; // + 32 * kb

    // dW ownership
    const int grp = wave / GROUP, pos = wave % GROUP;
    const int ta = (GROUP == 4) ? (pos >> 1) : 0, tb = (GROUP == 4) ? (pos & 1) : 0;
    // transposing-load source address of this lane inside a staged tile: row e_s (+4 for the second
    // load) of the 8-row half h, 4 consecutive features starting at 16*(G%2) + 4*qs of a 32-feature tile
    const int G = lane >> 4, e_s = (lane & 15) >> 2, qs = lane & 3;
    const int tr_row = 8 * h + e_s;
    const int tr_col = 16 * (G & 1) + 4 * qs;
    const bool tr_dead = (W == 16) && (G & 1); // features 16..31 do not exist at width 16

    f32x16 dWacc[N_MATS];
#pragma unroll
    for (int l = 0; l < N_MATS; ++l) dWacc[l] = f32x16{};
    float loss_local = 0.0f;

    const long long n_tiles = (M + 31) / 32;
    const long long tiles_per_round = (long long)gridDim.x * S::WAVES;
    const long long rounds = (n_tiles + tiles_per_round - 1) / tiles_per_round;

    for (long long round = 0; round < rounds; ++round) {
        const long long tile = (round * gridDim.x + blockIdx.x) * S::WAVES + wave;
        const long long row = tile * 32 + j;
        const bool valid = row < M;

        // ---------------- forward: activations of every layer stay in registers ----------------
        vec8 acts[N_MATS + 1][NK];
        TL::load(acts[0], x, row, h, valid);
        f32x16 acc[NI];
#pragma unroll
        for (int l = 0; l < N_MATS; ++l) {
            TL::template matmul<true>(acc, acts[l], lds_wf, lds_wf, l, lane);
            TL::repack_rt(acts[l + 1], acc, (l == N_MATS - 1) ? out_act : act);
        }
        if (y_out) TL::store(acts[N_MATS], y_out, row, h, valid);

        // ---------------- L2 loss and its gradient (include/losses/l2.h:19-25) ------------------
        vec8 cur[NK];
#pragma unroll
        for (int kb = 0; kb < NK; ++kb) {
            f32x8 g;
            if (valid) {
                const float4 *tp = reinterpret_cast<const float4 *>(targets + row * W + 16 * kb + 8 * h);
                const float4 t0 = tp[0], t1 = tp[1];
                const float tv[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float yv = (float)acts[N_MATS][kb][e];
                    const float diff = yv - tv[e];
                    loss_local += diff * diff * inv_n;
                    g[e] = as_fp32(loss_scale * 2 * diff * inv_n);
                }
            } else {
                g = f32x8{};
            }
            cur[kb] = __builtin_convertvector(g, vec8); // rounded to T exactly as the loss kernel stores it
            // derivative of the output activation on the T tile (kernel_esimd.h:193-201)
            if (out_act != TNN_ACT_NONE) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float gv = (float)cur[kb][e], f = (float)acts[N_MATS][kb][e];
                    g[e] = (out_act == TNN_ACT_RELU) ? ((f <= 0.0f) ? 0.0f : gv) : as_fp32(gv * (f * (1.0f - f)));
                }
                cur[kb] = __builtin_convertvector(g, vec8);
            }
        }

        // ---------------- backward: dW_l and delta_{l-1}, layer by layer ------------------------
#pragma unroll
        for (int l = N_MATS - 1; l >= 0; --l) {
            // stage delta_l and a_l row-major for the transposed reads
#pragma unroll
            for (int kb = 0; kb < NK; ++kb) {
                *reinterpret_cast<vec8 *>(my_d + wr_off + 32 * kb) = cur[kb];
                *reinterpret_cast<vec8 *>(my_a + wr_off + 32 * kb) = acts[l][kb];
            }
            __syncthreads();
#pragma unroll
            for (int q = 0; q < GROUP * 2; ++q) {
                const int src_wave = grp * GROUP + (q >> 1);
                const unsigned char *sd = stage + (size_t)(src_wave * 2 + 0) * S::TILE_BYTES;
                const unsigned char *sa = stage + (size_t)(src_wave * 2 + 1) * S::TILE_BYTES;
                const int r0 = (16 * (q & 1) + tr_row) * S::PITCH;
                const int r1 = r0 + 4 * S::PITCH;
                vec8 A = tr_load8<T>(sd, r0 + (32 * ta + tr_col) * 2, r1 + (32 * ta + tr_col) * 2);
                vec8 B = tr_load8<T>(sa, r0 + (32 * tb + tr_col) * 2, r1 + (32 * tb + tr_col) * 2);
                if (tr_dead) {
                    A = vec8{};
                    B = vec8{};
                }
                dWacc[l] = Storage<T>::mfma(A, B, dWacc[l]);
            }
            // delta_{l-1} (or dL/dx) while the other waves finish reading
            if (l > 0) {
                TL::template matmul<true>(acc, cur, lds_wb, lds_wb, l, lane);
                if (act == TNN_ACT_RELU)
                    TL::template bwd_repack<TNN_ACT_RELU>(cur, acc, acts[l]);
                else if (act == TNN_ACT_SIGMOID)
                    TL::template bwd_repack<TNN_ACT_SIGMOID>(cur, acc, acts[l]);
                else
                    TL::template repack<TNN_ACT_NONE>(cur, acc);
            } else if (dx_out) {
                TL::template matmul<true>(acc, cur, lds_wb, lds_wb, 0, lane);
                TL::template repack<TNN_ACT_NONE>(cur, acc);
                TL::store(cur, dx_out, row, h, valid);
            }
            __syncthreads(); // staged tiles are free again
        }
    }

    // ---------------- per-workgroup partials: sum the groups in a fixed order -------------------
    // (the whole LDS is reused as one fp32 [N_MATS][W][W] buffer; the loop above ended with a barrier)
    float *red = reinterpret_cast<float *>(smem_raw);
    for (int g = 0; g < S::N_GROUPS; ++g) {
        if (grp == g) {
#pragma unroll
            for (int l = 0; l < N_MATS; ++l) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int n = 32 * ta + 8 * (r >> 2) + 4 * h + (r & 3);
                    const int k = 32 * tb + j;
                    if (n < W && k < W) {
                        float *p = red + ((size_t)l * W + n) * W + k;
                        *p = (g == 0) ? dWacc[l][r] : *p + dWacc[l][r];
                    }
                }
            }
        }
        __syncthreads();
    }
    float *out = partials + (size_t)blockIdx.x * N_MATS * W * W;
    for (int idx = threadIdx.x; idx < N_MATS * W * W; idx += kFwdThreads) out[idx] = red[idx];

    // loss: wave sum, then the 8 wave sums in order
    __syncthreads();
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) loss_local += __shfl_down(loss_local, off, 64);
    if (lane == 0) red[wave] = loss_local;
    __syncthreads();
    if (threadIdx.x == 0) {
        float s = 0.0f;
        for (int w = 0; w < S::WAVES; ++w) s += red[w];
        loss_partials[blockIdx.x] = s;
    }
}

// Sums the per-workgroup partials in a fixed order. One thread per dW element; thread 0 of block 0
// also sums the loss partials.
template <typename T>
__global__ void train_reduce_kernel(const float *__restrict__ partials, const float *__restrict__ loss_partials, int n_partials,
                                    int n_elems, T *__restrict__ dW_T, float *__restrict__ dW_f32, float *__restrict__ loss_sum) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < n_elems) {
        float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
        int p = 0;
        for (; p + 3 < n_partials; p += 4) {
            s0 += partials[(size_t)(p + 0) * n_elems + idx];
            s1 += partials[(size_t)(p + 1) * n_elems + idx];
            s2 += partials[(size_t)(p + 2) * n_elems + idx];
            s3 += partials[(size_t)(p + 3) * n_elems + idx];
        }
        for (; p < n_partials; ++p) s0 += partials[(size_t)p * n_elems + idx];
        const float s = (s0 + s1) + (s2 + s3);
        if (dW_f32)
            dW_f32[idx] = s;
        else
            dW_T[idx] = (T)s;
    }
    if (loss_sum && idx == 0) {
        float s = 0.0f;
        for (int p = 0; p < n_partials; ++p) s += loss_partials[p];
        *loss_sum = s;
    }
}

// -------------------------------------------------------------------------------------------------
struct FusedPlan {
    bool supported;
    int grid;
    size_t lds;
    size_t partial_bytes; // fp32 [grid][n_mats][W][W]
    size_t loss_bytes;    // fp32 [grid]
};

static constexpr size_t kMaxLds = 160 * 1024;

template <int W> static FusedPlan plan_w(int n_mats, size_t M, int n_cu) {
    FusedPlan p;
    typedef TrainShape<W> S;
    p.lds = S::lds_bytes(n_mats);
    // the layer loop is unrolled: register budget bounds the depth (activations of all layers are live)
    const int max_mats = (W == 64) ? 5 : 6;
    p.supported = n_mats >= 2 && n_mats <= max_mats && p.lds <= kMaxLds;
    const long long n_tiles = ((long long)M + 31) / 32;
    long long g = (n_tiles + S::WAVES - 1) / S::WAVES;
    if (g > n_cu) g = n_cu;
    if (g < 1) g = 1;
    p.grid = (int)g;
    p.partial_bytes = (size_t)p.grid * n_mats * W * W * sizeof(float);
    p.loss_bytes = (((size_t)p.grid * sizeof(float)) + 255) & ~(size_t)255;
    return p;
}

static FusedPlan fused_plan(const tnn_mlp_desc *d, size_t M) {
    const DeviceInfo &di = device_info();
    const int n_cu = di.ok ? di.n_cu : 256;
    const int n_mats = d->n_hidden_layers + 1;
    switch (d->width) {
    case 16: return plan_w<16>(n_mats, M, n_cu);
    case 32: return plan_w<32>(n_mats, M, n_cu);
    case 64: return plan_w<64>(n_mats, M, n_cu);
    default: {
        FusedPlan p{};
        p.supported = false;
        return p;
    }
    }
}

template <typename T, int W, int N_MATS>
static int launch_fused(const tnn_mlp_desc *d, const FusedPlan &p, const void *wf, const void *wb, const void *x,
                        const float *targets, float loss_scale, void *y, float *loss_sum, void *dW, int dW_is_fp32, void *dx,
                        size_t M, float *partials, float *loss_partials, hipStream_t s) {
    typedef typename Storage<T>::vec8 vec8;
    auto k = mlp_train_fused_kernel<T, W, N_MATS>;
    if (p.lds > 48 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void *>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)p.lds) != hipSuccess)
        return fail(TNN_ERR_HIP, "cannot reserve %zu bytes of LDS", p.lds);
    const float inv_n = 1.0f / (float)(M * W);
    hipLaunchKernelGGL(k, dim3(p.grid), dim3(kFwdThreads), p.lds, s, (const vec8 *)wf, (const vec8 *)wb, (const T *)x, targets, (T *)y,
                       (T *)dx, partials, loss_partials, d->activation, d->output_activation, loss_scale, inv_n, (long long)M);
    int rc = check_launch("mlp_train_fused_kernel");
    if (rc) return rc;
    const int n_elems = N_MATS * W * W;
    hipLaunchKernelGGL((train_reduce_kernel<T>), dim3((n_elems + 255) / 256), dim3(256), 0, s, partials, loss_partials, p.grid,
                       n_elems, dW_is_fp32 ? (T *)nullptr : (T *)dW, dW_is_fp32 ? (float *)dW : (float *)nullptr, loss_sum);
    return check_launch("train_reduce_kernel");
}

template <typename T, int W>
static int launch_fused_n(const tnn_mlp_desc *d, const FusedPlan &p, const void *wf, const void *wb, const void *x,
                          const float *targets, float loss_scale, void *y, float *loss_sum, void *dW, int dW_is_fp32, void *dx,
                          size_t M, float *partials, float *loss_partials, hipStream_t s) {
#define TNN_CASE(N)                                                                                                      \
    case N: return launch_fused<T, W, N>(d, p, wf, wb, x, targets, loss_scale, y, loss_sum, dW, dW_is_fp32, dx, M, partials, loss_partials, s)
    switch (d->n_hidden_layers + 1) {
        TNN_CASE(2);
        TNN_CASE(3);
        TNN_CASE(4);
        TNN_CASE(5);
    case 6:
        if constexpr (W < 64)
            return launch_fused<T, W, 6>(d, p, wf, wb, x, targets, loss_scale, y, loss_sum, dW, dW_is_fp32, dx, M, partials, loss_partials, s);
        break;
    }
#undef TNN_CASE
    return fail(TNN_ERR_UNSUPPORTED, "fused training step: depth not instantiated");
}

// Used by tnn_mlp_train_step_l2: returns TNN_ERR_UNSUPPORTED when the shape has no fused kernel.
int fused_train_step(const tnn_mlp_desc *d, const void *wf, const void *wb, const void *x, const float *targets, float loss_scale,
                     void *y, float *loss_sum, void *dW, int dW_is_fp32, void *dx, size_t M, void *ws, size_t ws_bytes, hipStream_t s) {
    const FusedPlan p = fused_plan(d, M);
    if (!p.supported) return TNN_ERR_UNSUPPORTED;
    const size_t need = p.partial_bytes + p.loss_bytes + 512;
    if (!ws || ws_bytes < need) return fail(TNN_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", ws_bytes, need);
    uintptr_t base = (reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255;
    float *loss_partials = reinterpret_cast<float *>(base);
    float *partials = reinterpret_cast<float *>(base + p.loss_bytes);
    if (d->dtype == TNN_BF16) {
        switch (d->width) {
        case 16: return launch_fused_n<bf16_t, 16>(d, p, wf, wb, x, targets, loss_scale, y, loss_sum, dW, dW_is_fp32, dx, M, partials, loss_partials, s);
        case 32: return launch_fused_n<bf16_t, 32>(d, p, wf, wb, x, targets, loss_scale, y, loss_sum, dW, dW_is_fp32, dx, M, partials, loss_partials, s);
        default: return launch_fused_n<bf16_t, 64>(d, p, wf, wb, x, targets, loss_scale, y, loss_sum, dW, dW_is_fp32, dx, M, partials, loss_partials, s);
        }
    }
    switch (d->width) {
    case 16: return launch_fused_n<fp16_t, 16>(d, p, wf, wb, x, targets, loss_scale, y, loss_sum, dW, dW_is_fp32, dx, M, partials, loss_partials, s);
    case 32: return launch_fused_n<fp16_t, 32>(d, p, wf, wb, x, targets, loss_scale, y, loss_sum, dW, dW_is_fp32, dx, M, partials, loss_partials, s);
    default: return launch_fused_n<fp16_t, 64>(d, p, wf, wb, x, targets, loss_scale, y, loss_sum, dW, dW_is_fp32, dx, M, partials, loss_partials, s);
    }
}

// 0 when the shape has no fused kernel
size_t fused_train_workspace_bytes(const tnn_mlp_desc *d, size_t M) {
    const FusedPlan p = fused_plan(d, M);
    return p.supported ? p.partial_bytes + p.loss_bytes + 512 : 0;
}

} // namespace tnn
