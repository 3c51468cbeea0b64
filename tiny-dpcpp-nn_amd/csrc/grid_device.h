// Device-side pieces of the multi-resolution grid encoding shared by the stand-alone encoding kernels and the
// kernel that feeds the encoding straight into the fused MLP: per-level constants, the index functions, and the
// evaluation of one 16-byte piece of an encoded row.
//
// Reference behaviour being reproduced: include/encodings/grid.h:37-135 (kernel_grid),
// include/common/common_device.h:700-775 (hashes, grid_index, grid_scale, grid_resolution).
#pragma once

#include "tnn_internal.h"

namespace tnn {

struct GridLevels {
    uint32_t offset[TNN_GRID_MAX_LEVELS];  // entries
    uint32_t size[TNN_GRID_MAX_LEVELS];    // entries in the level ("hashmap_size")
    float scale[TNN_GRID_MAX_LEVELS];
    uint32_t resolution[TNN_GRID_MAX_LEVELS];
    // bits 0-3: number of dimensions that enter the strided index; bit 4: level is hashed;
    // bit 5: size is a power of two
    uint32_t flags[TNN_GRID_MAX_LEVELS];
};

struct GridParams {
    uint32_t n_levels;
    uint32_t hash_type;
    uint32_t interpolation;
    uint32_t padded_width;
};

// The buffer of tnn_grid_order_points (grid_order.hip): M records of 16 bytes, padded to 256 bytes, then the first position
// of each of the 4096 coarse cells of the order (uint32, key order), which the scatter over ordered points reads.
inline size_t order_record_bytes(size_t M) { return (M * 16 + 255) & ~(size_t)255; }

// Host side (grid.hip): validation of a descriptor, and of a call (include/encodings/grid.h:665-677) together with
// the per-level constants the kernels take.
int check_grid_desc(const tnn_grid_desc *d);
int grid_common(const tnn_grid_desc *desc, uint32_t padded_width, size_t M, GridLevels *lv, GridParams *gp);

template <int D> __device__ __forceinline__ uint32_t hash_pos(const uint32_t (&p)[D], uint32_t hash_type) {
    // include/common/common_device.h:713-729
    constexpr uint32_t prime[7] = {1958374283u, 2654435761u, 805459861u, 3674653429u, 2097192037u, 1434869437u, 2165219737u};
    constexpr uint32_t coherent[7] = {1u, 2654435761u, 805459861u, 3674653429u, 2097192037u, 1434869437u, 2165219737u};
    constexpr uint32_t reversed[7] = {2165219737u, 1434869437u, 2097192037u, 3674653429u, 805459861u, 2654435761u, 1958374283u};
    uint32_t r = 0;
    if (hash_type == TNN_HASH_COHERENT_PRIME) {
#pragma unroll
        for (int i = 0; i < D; ++i) r ^= p[i] * coherent[i];
    } else if (hash_type == TNN_HASH_PRIME) {
#pragma unroll
        for (int i = 0; i < D; ++i) r ^= p[i] * prime[i];
    } else if (hash_type == TNN_HASH_REVERSED_PRIME) {
#pragma unroll
        for (int i = 0; i < D; ++i) r ^= p[i] * reversed[i];
    }
    return r; // Rng hashes to 0, as in common_device.h:738-740
}

template <int D>
__device__ __forceinline__ uint32_t level_index(const uint32_t (&p)[D], uint32_t size, uint32_t res, uint32_t flags,
                                                uint32_t hash_type) {
    uint32_t index;
    if (flags & 16u) {
        index = hash_pos<D>(p, hash_type);
    } else {
        const uint32_t dims_used = flags & 15u;
        uint32_t stride = 1;
        index = 0;
#pragma unroll
        for (int dim = 0; dim < D; ++dim) {
            if ((uint32_t)dim < dims_used) {
                index += p[dim] * stride;
                stride *= res;
            }
        }
    }
    if (flags & 32u) return index & (size - 1);
    return (index >= size) ? index % size : index;
}

// include/encodings/grid.h:73-93
template <int D>
__device__ __forceinline__ void cell_of(const float (&x)[D], float scale, uint32_t interpolation, uint32_t (&cell)[D],
                                        float (&frac)[D]) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
        float p = __builtin_fmaf(scale, x[d], 0.5f);
        const float t = floorf(p);
        cell[d] = (uint32_t)(int)t;
        p -= t;
        frac[d] = (interpolation == TNN_INTERP_SMOOTHSTEP) ? p * p * (3.0f - 2.0f * p) : p;
    }
}

template <typename P, int F> __device__ __forceinline__ void load_entry(const P *__restrict__ p, float (&v)[F]) {
    // F consecutive features of one entry, fetched as a single vector load
    typedef P vecF __attribute__((ext_vector_type(F)));
    if (F == 1) {
        v[0] = (float)p[0];
    } else {
        const vecF t = *reinterpret_cast<const vecF *>(p);
#pragma unroll
        for (int f = 0; f < F; ++f) v[f] = (float)t[f];
    }
}

template <typename O> __device__ __forceinline__ O to_out(float v) { return (O)v; }

// Constants of one level as a kernel reads them (from its scalar arguments or from LDS).
struct LevelConst {
    uint32_t offset, size, resolution, flags;
    float scale;
};

__device__ __forceinline__ LevelConst level_const(const GridLevels &lv, uint32_t l) {
    return LevelConst{lv.offset[l], lv.size[l], lv.resolution[l], lv.flags[l], lv.scale[l]};
}

// GL consecutive levels of one point: all gathers of the group (GL * 2^D independent loads) are issued before the
// first blend. r[gl * F + f] is the interpolated feature in fp32, blended in the corner order and with the fused
// multiply-add of include/encodings/grid.h:114-129 (nearest: the single value is copied, grid.h:104-109); levels
// from n_valid on load nothing and give 0.
template <int D, int F, typename P, int GL>
__device__ __forceinline__ void encode_levels(const LevelConst (&lc)[GL], int n_valid, const GridParams &gp, const float (&x)[D],
                                              const P *__restrict__ table, float (&r)[GL * F]) {
    float vals[GL][1 << D][F];
    float wts[GL][1 << D];
#pragma unroll
    for (int gl = 0; gl < GL; ++gl) {
        if (gl < n_valid) {
            const uint32_t size = lc[gl].size, res = lc[gl].resolution, flags = lc[gl].flags;
            const P *g = table + (size_t)lc[gl].offset * F;
            uint32_t cell[D];
            float frac[D];
            cell_of<D>(x, lc[gl].scale, gp.interpolation, cell, frac);
            if (gp.interpolation == TNN_INTERP_NEAREST) {
                const uint32_t idx = level_index<D>(cell, size, res, flags, gp.hash_type);
                load_entry<P, F>(g + (size_t)idx * F, vals[gl][0]);
                wts[gl][0] = 1.0f;
#pragma unroll
                for (int c = 1; c < (1 << D); ++c) {
                    wts[gl][c] = 0.0f;
#pragma unroll
                    for (int f = 0; f < F; ++f) vals[gl][c][f] = 0.0f;
                }
            } else {
#pragma unroll
                for (int c = 0; c < (1 << D); ++c) {
                    float weight = 1.0f;
                    uint32_t loc[D];
#pragma unroll
                    for (int d = 0; d < D; ++d) {
                        if ((c & (1 << d)) == 0) {
                            weight *= 1 - frac[d];
                            loc[d] = cell[d];
                        } else {
                            weight *= frac[d];
                            loc[d] = cell[d] + 1;
                        }
                    }
                    wts[gl][c] = weight;
                    const uint32_t idx = level_index<D>(loc, size, res, flags, gp.hash_type);
                    load_entry<P, F>(g + (size_t)idx * F, vals[gl][c]);
                }
            }
        }
    }
#pragma unroll
    for (int gl = 0; gl < GL; ++gl) {
#pragma unroll
        for (int f = 0; f < F; ++f) {
            float v = 0.0f;
            if (gl < n_valid) {
                if (gp.interpolation == TNN_INTERP_NEAREST) {
                    v = vals[gl][0][f];
                } else {
#pragma unroll
                    for (int c = 0; c < (1 << D); ++c) v = __builtin_fmaf(wts[gl][c], vals[gl][c][f], v);
                }
            }
            // pinned as an fp32 number: the caller narrows it afterwards (the reference rounds the fp32 sum, a second
            // rounding), and without this the last multiply-add and the narrowing may merge into one instruction that
            // rounds once
            r[gl * F + f] = as_fp32(v);
        }
    }
}

} // namespace tnn
