// Adam on the fp32 master weights of a fused MLP, one weight at a time, with the re-staging of the rounded
// weight into the packed and the two operand-order copies. Shared by the stand-alone update kernel and by the
// reduction kernel of the fused training step.
#pragma once

#include <cmath>

#include "tnn_internal.h"

namespace tnn {

struct AdamArgs {
    float *master, *m, *v; // fp32, packed parameter layout
    float grad_scale;      // gradients are multiplied by this first (1 / loss_scale)
    float step_size;       // lr / (1 - beta1^t)
    float bc2_sqrt;        // sqrt(1 - beta2^t)
    float beta1, beta2, eps;
    void *packed_T, *prep_fwd, *prep_bwd; // of the network's storage type; each may be null
    int W;
};

// torch.optim.Adam's arithmetic (no weight decay, no amsgrad): the bias corrections are evaluated in double on
// the host, once per step.
inline AdamArgs make_adam_args(float *master, float *m, float *v, float grad_scale, int step, float lr, float beta1, float beta2,
                               float eps, void *packed_T, void *prep_fwd, void *prep_bwd, int W) {
    const double bc1 = 1.0 - std::pow((double)beta1, step);
    const double bc2 = 1.0 - std::pow((double)beta2, step);
    AdamArgs a;
    a.master = master, a.m = m, a.v = v;
    a.grad_scale = grad_scale;
    a.step_size = (float)(lr / bc1);
    a.bc2_sqrt = (float)std::sqrt(bc2);
    a.beta1 = beta1, a.beta2 = beta2, a.eps = eps;
    a.packed_T = packed_T, a.prep_fwd = prep_fwd, a.prep_bwd = prep_bwd;
    a.W = W;
    return a;
}

// One weight's optimizer state, fetched ahead of the gradient it will be updated with.
struct AdamElement {
    int pidx; // position in the packed parameter layout
    float m, v, w;
};

// idx: position in the raw gradient layout, matrix l, [n = out][k = in].
__device__ __forceinline__ AdamElement adam_fetch_element(const AdamArgs &a, int idx) {
    const int W = a.W, per = W * W;
    const int l = idx / per, e = idx % per;
    const int n = e / W, k = e % W;
    AdamElement s;
    s.pidx = l * per + packed_coord(k, n, W);
    s.m = a.m[s.pidx], s.v = a.v[s.pidx], s.w = a.master[s.pidx];
    return s;
}

// g_raw: the gradient element at idx; s: what adam_fetch_element(a, idx) returned.
template <typename T> __device__ __forceinline__ void adam_apply_element(const AdamArgs &a, int idx, const AdamElement &s, float g_raw) {
    const int W = a.W, per = W * W;
    const int l = idx / per, e = idx % per;
    const int n = e / W, k = e % W;
    const int pidx = s.pidx;
    const float g = g_raw * a.grad_scale;
    const float mi = s.m + (1.0f - a.beta1) * (g - s.m);
    const float vi = a.beta2 * s.v + (1.0f - a.beta2) * g * g;
    a.m[pidx] = mi;
    a.v[pidx] = vi;
    const float denom = sqrtf(vi) / a.bc2_sqrt + a.eps;
    const float p = s.w - a.step_size * (mi / denom);
    a.master[pidx] = p;
    const T pt = (T)p;
    if (a.packed_T) static_cast<T *>(a.packed_T)[pidx] = pt;
    const int NI = (W + 31) / 32, NK = W / 16;
    if (a.prep_fwd) // product index n, contraction index k
        static_cast<T *>(a.prep_fwd)[(((size_t)l * NI + n / 32) * NK + k / 16) * 512 + (32 * ((k % 16) / 8) + swap23(n % 32)) * 8 + (k % 8)] = pt;
    if (a.prep_bwd) // product index k, contraction index n
        static_cast<T *>(a.prep_bwd)[(((size_t)l * NI + k / 32) * NK + n / 16) * 512 + (32 * ((n % 16) / 8) + swap23(k % 32)) * 8 + (n % 8)] = pt;
}

template <typename T> __device__ __forceinline__ void adam_update_element(const AdamArgs &a, int idx, float g_raw) {
    adam_apply_element<T>(a, idx, adam_fetch_element(a, idx), g_raw);
}

// What follows the main kernel of the fused training step.
struct TrainTail {
    bool use_adam = false;       // apply Adam to the reduced gradients inside the reduction kernel
    AdamArgs adam{};
    hipEvent_t main_done = nullptr; // recorded between the main kernel and the reduction when not null
    void *dW = nullptr;             // launchers that have no dW argument of their own: where the reduced gradients go, if anywhere
    int dW_is_fp32 = 1;
};

} // namespace tnn
