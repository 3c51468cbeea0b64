// Device-side building blocks shared by the fused MLP kernels (gfx950): the per-wave 32-row tile in
// MFMA B-operand order, the weight-fragment product, and the activation / rounding steps.
//
// Register layout: lane (j = lane % 32, h = lane / 32) owns batch row j of the wave's tile; for every
// block kb of 16 features it holds the 8 features 16*kb + 8*h + [0, 8): one aligned 16-byte piece of
// the row-major row. Loads, stores and MFMA B operands all use this layout.
#pragma once

#include "tnn_internal.h"

namespace tnn {

constexpr int kFwdThreads = 512; // 8 waves per workgroup share one LDS copy of the weights
constexpr int kWaveSize = 64;

// ------------------------------------------------------------------------------------------
// Device helpers
// ------------------------------------------------------------------------------------------

template <int ACT> __device__ __forceinline__ float act_f32(float v) {
    if (ACT == TNN_ACT_RELU) return fmaxf(v, 0.0f);
    if (ACT == TNN_ACT_SIGMOID) return __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    return v;
}

// Accumulator half (8 fp32 of one 32x32 tile) -> activation -> 8 values of T.
// ReLU before or after the rounding gives the same value (rounding keeps the sign).
template <typename T, int ACT, int HALF>
__device__ __forceinline__ typename Storage<T>::vec8 act_convert(const f32x16 &c) {
    f32x8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = act_f32<ACT>(c[HALF * 8 + e]);
    return __builtin_convertvector(v, typename Storage<T>::vec8);
}

// Backward: fp32 accumulator, masked / scaled by the stored forward activation, then rounded.
template <typename T, int ACT, int HALF>
__device__ __forceinline__ typename Storage<T>::vec8 bwd_convert(const f32x16 &c,
                                                                 const typename Storage<T>::vec8 &fwd) {
    f32x8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float t = c[HALF * 8 + e];
        const float f = (float)fwd[e];
        if (ACT == TNN_ACT_RELU) t = (f <= 0.0f) ? 0.0f : t;
        if (ACT == TNN_ACT_SIGMOID) t = as_fp32(t * (f * (1.0f - f)));
        v[e] = t;
    }
    return __builtin_convertvector(v, typename Storage<T>::vec8);
}

template <typename T, int W> struct Tile {
    static constexpr int NK = W / 16;
    static constexpr int NI = (W + 31) / 32;
    typedef typename Storage<T>::vec8 vec8;

    // Row-major row `row` of an M x W matrix -> the lane's NK 16-byte pieces.
    static __device__ __forceinline__ void load(vec8 (&r)[NK], const T *__restrict__ base, long long row, int h,
                                                bool valid) {
        const vec8 *p = reinterpret_cast<const vec8 *>(base + row * W) + h;
#pragma unroll
        for (int kb = 0; kb < NK; ++kb) {
            if (valid)
                r[kb] = p[2 * kb];
            else
                r[kb] = vec8{};
        }
    }
    static __device__ __forceinline__ void store(const vec8 (&r)[NK], T *__restrict__ base, long long row, int h,
                                                 bool valid) {
        vec8 *p = reinterpret_cast<vec8 *>(base + row * W) + h;
        if (valid) {
#pragma unroll
            for (int kb = 0; kb < NK; ++kb) p[2 * kb] = r[kb];
        }
    }

    // acc[a] = sum_kb frag(l, a, kb) * b[kb]
    template <bool W_IN_LDS>
    static __device__ __forceinline__ void matmul(f32x16 (&acc)[NI], const vec8 (&b)[NK], const vec8 *__restrict__ lds_w,
                                                  const vec8 *__restrict__ glb_w, int l, int lane) {
        const vec8 *w = (W_IN_LDS ? lds_w : glb_w) + (size_t)l * (NI * NK * kWaveSize) + lane;
#pragma unroll
        for (int a = 0; a < NI; ++a) acc[a] = f32x16{};
#pragma unroll
        for (int kb = 0; kb < NK; ++kb) {
#pragma unroll
            for (int a = 0; a < NI; ++a) {
                const vec8 frag = w[(a * NK + kb) * kWaveSize];
                acc[a] = Storage<T>::mfma(frag, b[kb], acc[a]);
            }
        }
    }

    template <int ACT> static __device__ __forceinline__ void repack(vec8 (&r)[NK], const f32x16 (&acc)[NI]) {
#pragma unroll
        for (int a = 0; a < NI; ++a) {
            r[2 * a] = act_convert<T, ACT, 0>(acc[a]);
            if (2 * a + 1 < NK) r[2 * a + 1] = act_convert<T, ACT, 1>(acc[a]);
        }
    }
    static __device__ __forceinline__ void repack_rt(vec8 (&r)[NK], const f32x16 (&acc)[NI], int act) {
        if (act == TNN_ACT_RELU)
            repack<TNN_ACT_RELU>(r, acc);
        else if (act == TNN_ACT_SIGMOID)
            repack<TNN_ACT_SIGMOID>(r, acc);
        else
            repack<TNN_ACT_NONE>(r, acc);
    }

    template <int ACT>
    static __device__ __forceinline__ void bwd_repack(vec8 (&r)[NK], const f32x16 (&acc)[NI], const vec8 (&fwd)[NK]) {
#pragma unroll
        for (int a = 0; a < NI; ++a) {
            r[2 * a] = bwd_convert<T, ACT, 0>(acc[a], fwd[2 * a]);
            if (2 * a + 1 < NK) r[2 * a + 1] = bwd_convert<T, ACT, 1>(acc[a], fwd[2 * a + 1 < NK ? 2 * a + 1 : 0]);
        }
    }
};

template <typename T, int W>
__device__ __forceinline__ void stage_weights(typename Storage<T>::vec8 *lds_w,
                                              const typename Storage<T>::vec8 *__restrict__ glb_w, int n_mats) {
    constexpr int per_mat = Tile<T, W>::NI * Tile<T, W>::NK * kWaveSize;
    const int n = n_mats * per_mat;
    for (int f = threadIdx.x; f < n; f += blockDim.x) lds_w[f] = glb_w[f];
    __syncthreads();
}


struct DeviceInfo {
    int n_cu = 0;
    size_t max_lds = 0;
    bool ok = false;
};
const DeviceInfo &device_info();

inline size_t prepared_elems(const tnn_mlp_desc *d) {
    const int W = d->width, NI = (W + 31) / 32, NK = W / 16;
    return (size_t)(d->n_hidden_layers + 1) * NI * NK * 512;
}

} // namespace tnn
