// Multi-resolution hash-grid encoding for gfx950: forward gather + N-linear interpolation,
// backward scatter-add into an fp32 gradient table.
//
// Reference behaviour being reproduced: include/encodings/grid.h:37-135 (kernel_grid),
// :137-245 (kernel_grid_backward), :588-659 (offset table), :682-694 (zero padding of the output),
// include/common/common_device.h:700-775 (hashes, grid_index, grid_scale, grid_resolution).
//
// One thread owns one point and walks all levels: the coordinates are read once, every corner of a
// level is gathered before the blend (2^D independent loads in flight), and the whole encoded row is
// written as contiguous 16-byte pieces. Per-level constants (scale, resolution, table offset, size,
// how many dimensions enter the dense index, whether the level is hashed) are evaluated once on the
// host and reach the kernel as scalar kernel arguments; no thread evaluates exp2.
#include "grid_device.h"

#include <algorithm>
#include <cmath>
#include <cstring>

namespace tnn {

// include/common/common_device.h:745-765 evaluated for the loop bounds only: the stride sequence
// depends on (resolution, size, n_dims) and not on the position.
static void fill_levels(const tnn_grid_desc *d, GridLevels *lv) {
    for (uint32_t l = 0; l < d->n_levels; ++l) {
        const uint32_t size = d->offsets[l + 1] - d->offsets[l];
        lv->offset[l] = d->offsets[l];
        lv->size[l] = size;
        lv->scale[l] = d->scales[l];
        lv->resolution[l] = d->resolutions[l];
        uint32_t stride = 1, dims_used = 0;
        for (uint32_t dim = 0; dim < d->n_dims && stride <= size; ++dim) {
            ++dims_used;
            stride *= d->resolutions[l];
        }
        const bool hashed = (d->grid_type == TNN_GRID_HASH) && (size < stride);
        const bool pow2 = (size & (size - 1)) == 0;
        lv->flags[l] = dims_used | (hashed ? 16u : 0u) | (pow2 ? 32u : 0u);
    }
}

constexpr int kGridThreads = 256;


// Levels are processed in groups whose outputs fill one 16-byte piece of the encoded row: all gathers of a
// group (GL * 2^D independent loads) are issued before the first blend, and the row is written in whole
// 16-byte pieces (a per-level 4-byte store turns into a 32-byte masked write at the memory controller).
template <int D, int F, typename P, typename O>
__global__ void __launch_bounds__(kGridThreads)
    grid_forward_kernel(const GridLevels lv, const GridParams gp, const float *__restrict__ xin, const float4 *__restrict__ order,
                        const P *__restrict__ table, O *__restrict__ out, long long M) {
    constexpr int PER16 = 16 / (int)sizeof(O);            // outputs per 16-byte piece
    constexpr int GL = (PER16 / F) > 0 ? (PER16 / F) : 1; // levels per group (F = 8 with fp32 output: 1 level, 2 pieces)
    constexpr int NOUT = GL * F;
    typedef O ovec __attribute__((ext_vector_type(NOUT)));
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= M) return;
    // In cell order (grid_order.hip) thread i takes the i-th record, coordinates and row number, instead of row i.
    float x[D];
    long long row = i;
    if (order) {
        const float4 r = order[i];
        x[0] = r.x;
        x[1] = r.y;
        if (D > 2) x[D - 1] = r.z;
        row = (long long)__float_as_uint(r.w);
    } else {
#pragma unroll
        for (int d = 0; d < D; ++d) x[d] = xin[i * D + d];
    }
    O *orow = out + row * gp.padded_width;
    const bool row_aligned = ((gp.padded_width * sizeof(O)) % 16 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15) == 0);

    // The first kHeld pieces of a row (128 bytes with 16-byte pieces) are kept in registers and stored together when the
    // last of them is done, so that a row's pieces reach L2 back to back and leave it as one write; pieces computed
    // thousands of cycles apart would each sit in L2 as a partly written line among the table's lines.
    constexpr int kHeld = (NOUT * sizeof(O) == 16) ? 8 : 0;
    ovec held[kHeld > 0 ? kHeld : 1];
    auto do_group = [&](const uint32_t l0, ovec &o) __attribute__((always_inline)) {
        LevelConst lc[GL];
#pragma unroll
        for (int gl = 0; gl < GL; ++gl) lc[gl] = level_const(lv, (l0 + gl < gp.n_levels) ? l0 + gl : l0);
        const int n_valid = (int)((gp.n_levels - l0 < (uint32_t)GL) ? gp.n_levels - l0 : (uint32_t)GL);
        float r[NOUT];
        encode_levels<D, F, P, GL>(lc, n_valid, gp, x, table, r);
#pragma unroll
        for (int e = 0; e < NOUT; ++e) o[e] = to_out<O>(r[e]);
    };
    auto store_group = [&](const uint32_t l0, const ovec &o) __attribute__((always_inline)) {
        const uint32_t col0 = l0 * F;
        if (row_aligned && l0 + GL <= gp.n_levels) {
            if constexpr (NOUT * sizeof(O) == 16) {
                *reinterpret_cast<ovec *>(orow + col0) = o;
            } else { // F = 8 with fp32 output: two 16-byte pieces
#pragma unroll
                for (int e = 0; e < NOUT; ++e) orow[col0 + e] = o[e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < NOUT; ++e)
                if (l0 + e / F < gp.n_levels) orow[col0 + e] = o[e];
        }
    };
#pragma unroll
    for (int p = 0; p < kHeld; ++p)
        if ((uint32_t)(p * GL) < gp.n_levels) do_group((uint32_t)(p * GL), held[p]);
#pragma unroll
    for (int p = 0; p < kHeld; ++p)
        if ((uint32_t)(p * GL) < gp.n_levels) store_group((uint32_t)(p * GL), held[p]);
    for (uint32_t l0 = kHeld * GL; l0 < gp.n_levels; l0 += GL) {
        ovec o;
        do_group(l0, o);
        store_group(l0, o);
    }
    // zero padding of the row (include/encodings/grid.h:682-694), in 16-byte pieces where the row allows it
    uint32_t c = gp.n_levels * F;
    if (row_aligned) {
        typedef O zvec __attribute__((ext_vector_type(PER16)));
        for (; c < gp.padded_width && (c % PER16) != 0; ++c) orow[c] = to_out<O>(0.0f);
        for (; c + PER16 <= gp.padded_width; c += PER16) *reinterpret_cast<zvec *>(orow + c) = zvec{};
    }
    for (; c < gp.padded_width; ++c) orow[c] = to_out<O>(0.0f);
}

template <int D>
__global__ void __launch_bounds__(kGridThreads)
    grid_indices_kernel(const GridLevels lv, const GridParams gp, const float *__restrict__ xin, uint32_t *__restrict__ out,
                        long long M) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= M) return;
    float x[D];
#pragma unroll
    for (int d = 0; d < D; ++d) x[d] = xin[i * D + d];
    for (uint32_t l = 0; l < gp.n_levels; ++l) {
        uint32_t cell[D];
        float frac[D];
        cell_of<D>(x, lv.scale[l], gp.interpolation, cell, frac);
#pragma unroll
        for (int c = 0; c < (1 << D); ++c) {
            uint32_t loc[D];
#pragma unroll
            for (int d = 0; d < D; ++d) loc[d] = (c & (1 << d)) ? cell[d] + 1 : cell[d];
            out[(i * gp.n_levels + l) * (1 << D) + c] = level_index<D>(loc, lv.size[l], lv.resolution[l], lv.flags[l], gp.hash_type);
        }
    }
}

// Which levels the backward pass accumulates in LDS first, and how the 1-D grid is split between the two routes.
struct BackwardPlan {
    uint32_t n_small;          // levels whose whole gradient slice fits the LDS budget
    uint32_t small_blocks;     // workgroups per such level, each takes `chunk` consecutive points
    uint32_t chunk;
    uint32_t big_blocks;       // workgroups per other level, a group of lanes per point
    uint8_t small_level[TNN_GRID_MAX_LEVELS];
    uint8_t big_level[TNN_GRID_MAX_LEVELS];
    // Points in cell order only: levels too large for a private copy of the whole level, where a stretch of consecutive
    // points still lands on few enough cells for a private copy of the box around them (kMaxTiled such levels).
    uint32_t n_tiled;
    uint32_t budget;           // LDS bytes a workgroup may use
    uint32_t tiled_start[17]; // first workgroup of each such level among the tiled workgroups, and their total
    uint8_t tiled_level[16];
    uint8_t tiled_chunk_log2[16]; // a stretch of the level is 2^n consecutive points
    uint8_t tiled_pieces[16];     // workgroups per row of the order's coarse cells; they take the row's stretches in turn
    uint32_t bins_per_row;        // coarse cells in a row (64 in 2-D, 16 in 3-D), n_rows rows
    uint32_t n_rows;
};
constexpr uint32_t kMaxTiled = 16;
#ifndef TNN_BOXED_MIN_PER_CELL
#define TNN_BOXED_MIN_PER_CELL 0.3
#endif
constexpr double kBoxedMinPerCell = TNN_BOXED_MIN_PER_CELL; // points of the batch per cell of a level, at least, for the boxed route

constexpr int kGridWave = 64;                    // lanes of a wave
constexpr int kBwdThreads = 512;                 // the backward kernel's workgroups
constexpr int kDirectPasses = 8;                 // groups of kBwdThreads / lanes-per-point points a direct-route workgroup takes
constexpr uint32_t kPrivateLdsBytes = 64 * 1024; // LDS budget of a workgroup; two such workgroups fit a CU
// In cell order more levels take an LDS route, and the launch's LDS size holds for every workgroup, also for those of the
// direct route, which need none: four workgroups of 40 KiB fill a CU's wave slots.
constexpr uint32_t kPrivateLdsBytesOrdered = 40 * 1024;
constexpr uint32_t kPrivateChunk = 4096;         // points per workgroup on the LDS route

// Coordinates and row number of the i-th point: row i of x, or the i-th record of the cell order (grid_order.hip).
template <int D>
__device__ __forceinline__ long long load_point(const float *__restrict__ xin, const float4 *__restrict__ order, long long i, float (&x)[D]) {
    if (order) {
        const float4 r = order[i];
        x[0] = r.x;
        x[1] = r.y;
        if (D > 2) x[D - 1] = r.z;
        return (long long)__float_as_uint(r.w);
    }
#pragma unroll
    for (int d = 0; d < D; ++d) x[d] = xin[i * D + d];
    return i;
}

// Gradient contributions of one point to one level: visits (entry index, weight) of every corner.
template <int D, typename Fn>
__device__ __forceinline__ void for_each_corner(const float (&x)[D], float scale, uint32_t size, uint32_t res, uint32_t flags,
                                                uint32_t hash_type, uint32_t interpolation, Fn &&fn) {
    uint32_t cell[D];
    float frac[D];
    cell_of<D>(x, scale, interpolation, cell, frac);
    if (interpolation == TNN_INTERP_NEAREST) {
        fn(level_index<D>(cell, size, res, flags, hash_type), 1.0f);
        return;
    }
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
        fn(level_index<D>(loc, size, res, flags, hash_type), weight);
    }
}

typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

// Adds the F gradient values of one table entry. fp32 tables: one atomic per value (the reference's grad_t). fp16 tables:
// one packed atomic (global_atomic_pk_add_f16) per pair of features, half as many atomic operations.
template <int F> __device__ __forceinline__ void add_entry(float *entry, const float (&v)[F]) {
#pragma unroll
    for (int f = 0; f < F; ++f) unsafeAtomicAdd(entry + f, v[f]);
}
template <int F> __device__ __forceinline__ void add_entry(fp16_t *entry, const float (&v)[F]) {
    static_assert(F % 2 == 0, "packed fp16 gradients need an even number of features per level");
#pragma unroll
    for (int f = 0; f < F; f += 2) {
        const f16x2_t pair = {(fp16_t)v[f], (fp16_t)v[f + 1]};
        (void)__builtin_amdgcn_flat_atomic_fadd_v2f16(reinterpret_cast<f16x2_t *>(entry + f), pair);
    }
}

// Lanes over the features of one entry on the direct route: one per value for an fp32 table, one per packed pair for fp16.
template <int F, typename GT> struct BackwardLanes { static constexpr int FL = F; };
template <int F> struct BackwardLanes<F, fp16_t> { static constexpr int FL = F / 2; };

// Lane i of a row of 16 lanes reads lane i - N (row_shr) or i + N (row_shl) of the same row; lanes without such a
// neighbour keep their own value.
template <int N> __device__ __forceinline__ int row_shr(int v) {
    if constexpr (N >= 16) return v;
    else return __builtin_amdgcn_update_dpp(v, v, 0x110 + N, 0xf, 0xf, false);
}
template <int N> __device__ __forceinline__ int row_shl(int v) {
    if constexpr (N >= 16) return v;
    else return __builtin_amdgcn_update_dpp(v, v, 0x100 + N, 0xf, 0xf, false);
}
// One step of a segmented inclusive sum inside rows of 16 lanes: lanes whose run is still open take the sum STEP lanes up.
template <int STEP, int FV> __device__ __forceinline__ void segmented_step(float (&v)[FV], bool &open, int rl) {
    const bool open_up = row_shr<STEP>((int)open) != 0;
    const bool reach = rl >= STEP;
#pragma unroll
    for (int f = 0; f < FV; ++f) {
        const float up = __int_as_float(row_shr<STEP>(__float_as_int(v[f])));
        v[f] += (reach && open) ? up : 0.0f;
    }
    open = reach ? (open && open_up) : open;
}

// Scatter-add of dL/dy into the gradient table (include/encodings/grid.h:137-245 of the reference: float atomics,
// order not defined). Two routes inside one launch:
//   * small levels (the coarse ones, where every point of the batch lands on a few hundred entries and global
//     atomics queue up on the same addresses): a workgroup adds the contributions of a chunk of points into a
//     private copy of the level in LDS and then issues one global atomic per touched entry;
//   * the other levels: a group of lanes per (point, level), atomics straight to the table; workgroups of one level
//     are dispatched together, so its slice of the table is the hot one in L2.
template <int D, int F, typename G, typename GT>
__global__ void __launch_bounds__(kBwdThreads)
    grid_backward_kernel(const GridLevels lv, const GridParams gp, const BackwardPlan bp, const float *__restrict__ xin,
                         const float4 *__restrict__ order, const uint32_t *__restrict__ bin_start, const G *__restrict__ dLdy,
                         GT *__restrict__ grad, long long M) {
    extern __shared__ float priv[];
    const uint32_t n_small_blocks = bp.n_small * bp.small_blocks;
    // Workgroups start in the order of their numbers. Those of the LDS routes and those of the direct route are bound by
    // different things (LDS atomics; atomic requests to memory), so their numbers are interleaved in proportion: both kinds
    // are resident on every CU from the start, instead of one kind queueing behind the other.
    const uint32_t n_lds_blocks = n_small_blocks + bp.tiled_start[bp.n_tiled];
    // (Cell order only. In the caller's order the few long workgroups of the LDS route come first, as measured faster.)
    const uint32_t n_direct_before =
        order ? (uint32_t)(((unsigned long long)blockIdx.x * (gridDim.x - n_lds_blocks)) / gridDim.x) : (blockIdx.x < n_lds_blocks ? 0u : blockIdx.x - n_lds_blocks);
    const bool is_direct = order ? (uint32_t)(((unsigned long long)(blockIdx.x + 1) * (gridDim.x - n_lds_blocks)) / gridDim.x) != n_direct_before
                                 : blockIdx.x >= n_lds_blocks;
    const uint32_t lds_block = blockIdx.x - n_direct_before; // this workgroup's number among those of its kind
    if (!is_direct && lds_block < n_small_blocks) {
        const uint32_t l = bp.small_level[lds_block / bp.small_blocks];
        const uint32_t size = lv.size[l], res = lv.resolution[l], flags = lv.flags[l];
        const float scale = lv.scale[l];
        const uint32_t n = size * F;
        for (uint32_t e = threadIdx.x; e < n; e += kBwdThreads) priv[e] = 0.0f;
        __syncthreads();
        const long long first = (long long)(lds_block % bp.small_blocks) * bp.chunk;
        const long long last = first + bp.chunk < M ? first + bp.chunk : M;
        for (long long i = first + threadIdx.x; i < last; i += kBwdThreads) {
            float x[D];
            const long long row = load_point<D>(xin, order, i, x);
            float gy[F];
#pragma unroll
            for (int f = 0; f < F; ++f) gy[f] = (float)dLdy[row * gp.padded_width + l * F + f];
            for_each_corner<D>(x, scale, size, res, flags, gp.hash_type, gp.interpolation, [&](uint32_t idx, float w) {
#pragma unroll
                for (int f = 0; f < F; ++f) atomicAdd(&priv[idx * F + f], w * gy[f]);
            });
        }
        __syncthreads();
        GT *g = grad + (size_t)lv.offset[l] * F;
        for (uint32_t e = threadIdx.x; e < size; e += kBwdThreads) {
            float v[F];
            bool any = false;
#pragma unroll
            for (int f = 0; f < F; ++f) {
                v[f] = priv[e * F + f];
                any |= v[f] != 0.0f;
            }
            if (any) add_entry<F>(g + (size_t)e * F, v);
        }
        return;
    }
    if (!is_direct) {
        // Cell order, a level whose workgroups each take stretches of consecutive points of one row of the order's coarse
        // cells (grid_order.hip walks the coarse cells row by row, x fastest, and leaves the first position of every
        // coarse cell behind the records): such a stretch lies in a few neighbouring cells, so the corners it touches fill
        // a small box of the level's cells. The workgroup finds that box, accumulates in a private fp32 copy of it in LDS,
        // and adds every touched entry to the table once. A stretch whose box does not fit (points far apart: the bins of
        // the points outside the unit cube, a sparse region) adds to the table directly.
        const uint32_t tb = lds_block - n_small_blocks;
        uint32_t ti = 0;
        while (ti + 1 < bp.n_tiled && tb >= bp.tiled_start[ti + 1]) ++ti;
        const uint32_t l = bp.tiled_level[ti];
        const uint32_t chunk = 1u << bp.tiled_chunk_log2[ti], pieces = bp.tiled_pieces[ti];
        const uint32_t rowno = (tb - bp.tiled_start[ti]) / pieces, piece = (tb - bp.tiled_start[ti]) % pieces;
        const uint32_t size = lv.size[l], res = lv.resolution[l], flags = lv.flags[l];
        const float scale = lv.scale[l];
        const long long row_first = bin_start[rowno * bp.bins_per_row];
        const long long row_end = rowno + 1 < bp.n_rows ? (long long)bin_start[(rowno + 1) * bp.bins_per_row] : M;
        __shared__ int box_lo[D], box_hi[D];
        // lane L of wave w takes the points L * stripe + w + n_waves * k of the stretch: the lanes of an instruction are a
        // stripe apart and rarely in the same cell, where consecutive points would queue up on one LDS address
        constexpr uint32_t n_waves = kBwdThreads / kGridWave;
        const uint32_t stripe = chunk / kGridWave, wv = threadIdx.x / kGridWave, ln = threadIdx.x % kGridWave;
        const bool nearest = gp.interpolation == TNN_INTERP_NEAREST;
        GT *g = grad + (size_t)lv.offset[l] * F;
        for (long long first = row_first + (long long)piece * chunk; first < row_end; first += (long long)pieces * chunk) {
            const uint32_t count = (uint32_t)((first + chunk < row_end ? first + chunk : row_end) - first);
            __syncthreads(); // the box and the private copy of the stretch before are done with
            if (threadIdx.x < D) {
                box_lo[threadIdx.x] = 0x7fffffff;
                box_hi[threadIdx.x] = (int)0x80000000;
            }
            __syncthreads();
            int lo[D], hi[D];
#pragma unroll
            for (int d = 0; d < D; ++d) {
                lo[d] = 0x7fffffff;
                hi[d] = (int)0x80000000;
            }
            for (uint32_t k = wv; k < stripe; k += n_waves) {
                const uint32_t pl = ln * stripe + k;
                if (pl >= count) continue;
                float x[D];
                load_point<D>(xin, order, first + pl, x);
                uint32_t cell[D];
                float frac[D];
                cell_of<D>(x, scale, gp.interpolation, cell, frac);
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    const int c = (int)cell[d];
                    lo[d] = c < lo[d] ? c : lo[d];
                    hi[d] = c > hi[d] ? c : hi[d];
                }
            }
#pragma unroll
            for (int d = 0; d < D; ++d) {
#pragma unroll
                for (int off = kGridWave / 2; off > 0; off >>= 1) {
                    const int a = __shfl_xor(lo[d], off, kGridWave), b2 = __shfl_xor(hi[d], off, kGridWave);
                    lo[d] = a < lo[d] ? a : lo[d];
                    hi[d] = b2 > hi[d] ? b2 : hi[d];
                }
                if (ln == 0 && lo[d] <= hi[d]) {
                    atomicMin(&box_lo[d], lo[d]);
                    atomicMax(&box_hi[d], hi[d]);
                }
            }
            __syncthreads();
            long long n_local = 1;
            uint32_t ext[D];
#pragma unroll
            for (int d = 0; d < D; ++d) {
                lo[d] = box_lo[d];
                const long long e = (long long)box_hi[d] - lo[d] + (nearest ? 1 : 2); // the far corners are one cell further
                ext[d] = (uint32_t)e;
                n_local = (e <= 0 || n_local > (1ll << 40)) ? (1ll << 41) : n_local * e;
            }
            const bool fits = n_local * F * (long long)sizeof(float) <= (long long)bp.budget;
            if (fits) {
                for (uint32_t e = threadIdx.x; e < (uint32_t)n_local * F; e += kBwdThreads) priv[e] = 0.0f;
                __syncthreads();
            }
            for (uint32_t k = wv; k < stripe; k += n_waves) {
                const uint32_t pl = ln * stripe + k;
                if (pl >= count) continue;
                float x[D];
                const long long row = load_point<D>(xin, order, first + pl, x);
                float gy[F];
#pragma unroll
                for (int f = 0; f < F; ++f) gy[f] = (float)dLdy[row * gp.padded_width + l * F + f];
                uint32_t cell[D];
                float frac[D];
                cell_of<D>(x, scale, gp.interpolation, cell, frac);
#pragma unroll
                for (int c = 0; c < (1 << D); ++c) {
                    if (nearest && c > 0) break;
                    float weight = 1.0f;
                    uint32_t loc[D];
                    uint32_t local = 0, stride = 1;
#pragma unroll
                    for (int d = 0; d < D; ++d) {
                        const bool far = !nearest && (c & (1 << d));
                        weight *= nearest ? 1.0f : (far ? frac[d] : 1 - frac[d]); // the products of for_each_corner
                        loc[d] = far ? cell[d] + 1 : cell[d];
                        local += (uint32_t)((int)loc[d] - lo[d]) * stride;
                        stride *= ext[d];
                    }
                    if (fits) {
#pragma unroll
                        for (int f = 0; f < F; ++f) atomicAdd(&priv[local * F + f], weight * gy[f]);
                    } else {
                        float v[F];
#pragma unroll
                        for (int f = 0; f < F; ++f) v[f] = weight * gy[f];
                        add_entry<F>(g + (size_t)level_index<D>(loc, size, res, flags, gp.hash_type) * F, v);
                    }
                }
            }
            if (!fits) continue;
            __syncthreads();
            for (uint32_t e = threadIdx.x; e < (uint32_t)n_local; e += kBwdThreads) {
                float v[F];
                bool any = false;
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    v[f] = priv[e * F + f];
                    any |= v[f] != 0.0f;
                }
                if (!any) continue;
                uint32_t loc[D], rest = e;
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    loc[d] = (uint32_t)(lo[d] + (int)(rest % ext[d]));
                    rest /= ext[d];
                }
                add_entry<F>(g + (size_t)level_index<D>(loc, size, res, flags, gp.hash_type) * F, v);
            }
        }
        return;
    }
    // A group of 2 * FL neighbouring lanes owns one (point, level): lane (dx, fl) adds feature fl (fp16 table: the pair of
    // features fl) of the corners on side dx of the cell along the first dimension. The memory side retires atomic
    // requests per 32-byte sector, about 20 * 10^9 a second, however many lanes of one instruction fall into the sector:
    // the features of an entry always do, and the two corners along the first dimension are neighbouring entries
    // wherever that dimension enters the index unhashed or the hash leaves it in the low bits.
    constexpr int FL = BackwardLanes<F, GT>::FL, LPI = 2 * FL;
    const uint32_t b = n_direct_before;
    const uint32_t l = bp.big_level[b / bp.big_blocks];
    // kDirectPasses groups of points per workgroup, one after the other: a workgroup that ended after two atomics per lane
    // left the launch bound by the rate at which workgroups are dispatched
    GT *const g = grad + (size_t)lv.offset[l] * F + (threadIdx.x % FL) * (F / FL);
    const uint32_t size = lv.size[l], res = lv.resolution[l], flags = lv.flags[l];
    for (int pass = 0; pass < kDirectPasses; ++pass) {
    const long long i_raw = ((long long)(b % bp.big_blocks) * kDirectPasses + pass) * (kBwdThreads / LPI) + threadIdx.x / LPI;
    const bool live = i_raw < M;
    if (i_raw - threadIdx.x / LPI >= M) break; // the whole workgroup is past the end
    if (!live && !order) continue;
    const long long i = live ? i_raw : M - 1; // in cell order every lane stays for the exchange between lanes below
    const int dx = (threadIdx.x % LPI) / FL, fl = threadIdx.x % FL;
    float x[D];
    const long long row = load_point<D>(xin, order, i, x);
    constexpr int FV = F / FL; // values per lane: 1 (fp32 table) or 2 (fp16 table)
    float gy[FV];
#pragma unroll
    for (int f = 0; f < FV; ++f) gy[f] = live ? (float)dLdy[row * gp.padded_width + l * F + fl * FV + f] : 0.0f;
    uint32_t cell[D];
    float frac[D];
    cell_of<D>(x, lv.scale[l], gp.interpolation, cell, frac);
    if (gp.interpolation == TNN_INTERP_NEAREST) {
        if (dx == 0 && live) add_entry<FV>(g + (size_t)level_index<D>(cell, size, res, flags, gp.hash_type) * F, gy);
        continue;
    }
#pragma unroll
    for (int rest = 0; rest < (1 << (D - 1)); ++rest) {
        const int c = 2 * rest + dx; // same corner numbering and weight product as for_each_corner
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
        float v[FV];
#pragma unroll
        for (int f = 0; f < FV; ++f) v[f] = weight * gy[f];
        const uint32_t idx = level_index<D>(loc, size, res, flags, gp.hash_type);
        if (order) {
            // Points in cell order: neighbouring groups of lanes often hold the same entry. Runs of equal entries inside a row
            // of 16 lanes are summed first (a segmented sum over the lanes LPI apart, which hold the same side and feature
            // of the next points) and the last lane of a run adds the total: one atomic per run instead of one per point.
            // Lanes exchange through DPP row shifts, not through the LDS crossbar, which the workgroups of the LDS routes
            // on the same CU keep busy with their atomics. The order of the additions is not defined in the reference
            // either (grid.h:215-243).
            const int rl = (int)(threadIdx.x % 16);
            const uint32_t idx_prev = (uint32_t)row_shr<LPI>((int)idx);
            bool open = rl >= LPI && idx_prev == idx; // this lane's run starts further up than the steps so far have reached
            if constexpr (LPI < 16) {
                segmented_step<LPI, FV>(v, open, rl);
                if constexpr (2 * LPI < 16) segmented_step<2 * LPI, FV>(v, open, rl);
                if constexpr (4 * LPI < 16) segmented_step<4 * LPI, FV>(v, open, rl);
                if constexpr (8 * LPI < 16) segmented_step<8 * LPI, FV>(v, open, rl);
            }
            const uint32_t idx_next = (uint32_t)row_shl<LPI>((int)idx);
            const bool last = rl + LPI >= 16 || idx_next != idx;
            if (last) add_entry<FV>(g + (size_t)idx * F, v);
        } else {
            add_entry<FV>(g + (size_t)idx * F, v);
        }
    }
    }
}

__global__ void fill_zero_kernel(float4 *__restrict__ p, size_t n4, float *__restrict__ tail, size_t n_tail) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t k = i; k < n4; k += stride) p[k] = float4{0.f, 0.f, 0.f, 0.f};
    if (i < n_tail) tail[i] = 0.0f;
}

int check_grid_desc(const tnn_grid_desc *d) {
    if (!d) return fail(TNN_ERR_INVALID_ARGUMENT, "desc is NULL");
    if (d->n_dims != 2 && d->n_dims != 3) return fail(TNN_ERR_UNSUPPORTED, "GridEncoding: n_dims_to_encode %u (2 or 3 are built)", d->n_dims);
    if (d->n_levels == 0 || d->n_levels > TNN_GRID_MAX_LEVELS)
        return fail(TNN_ERR_INVALID_ARGUMENT, "GridEncoding: n_levels %u must be at most MAX_N_LEVELS %d", d->n_levels, TNN_GRID_MAX_LEVELS);
    const uint32_t F = d->n_features_per_level;
    if (F != 1 && F != 2 && F != 4 && F != 8) return fail(TNN_ERR_INVALID_ARGUMENT, "GridEncoding: n_features_per_level must be 1, 2, 4, or 8.");
    if (d->param_dtype != TNN_FP32 && d->param_dtype != TNN_FP16) return fail(TNN_ERR_UNSUPPORTED, "table dtype %u", d->param_dtype);
    if (d->grid_type > TNN_GRID_TILED || d->hash_type > TNN_HASH_RNG || d->interpolation > TNN_INTERP_SMOOTHSTEP)
        return fail(TNN_ERR_INVALID_ARGUMENT, "invalid grid / hash / interpolation type");
    return TNN_OK;
}

template <int D, int F, typename P>
static int launch_grid_forward_o(const GridLevels &lv, const GridParams &gp, const float *x, const float4 *order, const void *table,
                                 void *out, int out_dtype, size_t M, hipStream_t s) {
    const unsigned blocks = (unsigned)((M + kGridThreads - 1) / kGridThreads);
    switch (out_dtype) {
    case TNN_FP32:
        TNN_LAUNCH((grid_forward_kernel<D, F, P, float>), dim3(blocks), dim3(kGridThreads), 0, s, lv, gp, x, order, (const P *)table,
                           (float *)out, (long long)M);
        break;
    case TNN_BF16:
        TNN_LAUNCH((grid_forward_kernel<D, F, P, bf16_t>), dim3(blocks), dim3(kGridThreads), 0, s, lv, gp, x, order, (const P *)table,
                           (bf16_t *)out, (long long)M);
        break;
    case TNN_FP16:
        TNN_LAUNCH((grid_forward_kernel<D, F, P, fp16_t>), dim3(blocks), dim3(kGridThreads), 0, s, lv, gp, x, order, (const P *)table,
                           (fp16_t *)out, (long long)M);
        break;
    default: return fail(TNN_ERR_UNSUPPORTED, "out_dtype %d", out_dtype);
    }
    return check_launch("grid_forward_kernel");
}

template <int D, int F>
static int launch_grid_forward_p(const tnn_grid_desc *d, const GridLevels &lv, const GridParams &gp, const float *x, const float4 *order,
                                 const void *table, void *out, int out_dtype, size_t M, hipStream_t s) {
    if (d->param_dtype == TNN_FP32) return launch_grid_forward_o<D, F, float>(lv, gp, x, order, table, out, out_dtype, M, s);
    return launch_grid_forward_o<D, F, fp16_t>(lv, gp, x, order, table, out, out_dtype, M, s);
}

template <int D, int F, typename TAB>
static int launch_grid_backward_g(const GridLevels &lv, const GridParams &gp, const float *x, const float4 *order, const void *dLdy,
                                  int dy_dtype, TAB *grad, size_t M, hipStream_t s) {
    // A level goes the LDS route when its slice fits the budget and a chunk of points makes clearly more atomics
    // than the flush of the private copy does (chunk * 2^D contributions against `size` entries).
    BackwardPlan bp{};
    bp.chunk = kPrivateChunk;
    bp.budget = order ? kPrivateLdsBytesOrdered : kPrivateLdsBytes;
    bp.small_blocks = (uint32_t)((M + bp.chunk - 1) / bp.chunk);
    constexpr int per_block = kDirectPasses * kBwdThreads / (2 * BackwardLanes<F, TAB>::FL); // (point, level) pairs per workgroup on the direct route
    bp.big_blocks = (uint32_t)((M + per_block - 1) / per_block);
    const size_t per_chunk = (M < bp.chunk ? M : (size_t)bp.chunk) << (gp.interpolation == TNN_INTERP_NEAREST ? 0 : D);
    uint32_t n_big = 0, lds_bytes = 0;
    for (uint32_t l = 0; l < gp.n_levels; ++l) {
        const size_t bytes = (size_t)lv.size[l] * F * sizeof(float);
        // (in cell order only the coarsest levels: the box of a stretch is far smaller than a level from 8 KiB on)
        if (bytes <= (order ? 8192u : bp.budget) && per_chunk >= 2 * (size_t)lv.size[l]) {
            bp.small_level[bp.n_small++] = (uint8_t)l;
            if (bytes > lds_bytes) lds_bytes = (uint32_t)bytes;
        } else {
            bp.big_level[n_big++] = (uint8_t)l;
        }
    }
    // Cell order: of the other levels, those where a stretch of consecutive points of one row of the order's coarse cells
    // fills a box of the level's cells that fits the LDS budget take the boxed route, as long as the level has a point for
    // every few cells (beyond that a box holds hardly more than one contribution per entry and saves no atomics). The order
    // (grid_order.hip) walks a lattice of 64^2 (16^3) coarse cells row by row, x fastest: with the points spread evenly a
    // row holds M / 64 (M / 256) of them, and a stretch of C of these spans that share of the level's width plus a coarse
    // cell, and one coarse cell in the other dimensions. A stretch that breaks the estimate is caught in the kernel.
    const uint32_t *bin_start = nullptr;
    if (order && gp.n_levels > 0 && gp.interpolation != TNN_INTERP_NEAREST) {
        bin_start = reinterpret_cast<const uint32_t *>(reinterpret_cast<const char *>(order) + order_record_bytes(M));
        bp.bins_per_row = (D == 2) ? 64 : 16;
        bp.n_rows = 4096 / bp.bins_per_row;
        const double per_row = (double)M / bp.n_rows, coarse = (double)bp.bins_per_row;
        uint32_t kept = 0;
        for (uint32_t i = 0; i < n_big; ++i) {
            const uint32_t l = bp.big_level[i];
            const double R = (double)lv.resolution[l];
            const double per_cell = (double)M / std::pow(R, (double)D);
            int chunk_log2 = -1;
            // (short stretches: many workgroups of some ten microseconds each spread over the CUs far more evenly than few long ones)
            for (int c = 10; c >= 9 && chunk_log2 < 0 && bp.n_tiled < kMaxTiled && per_cell >= kBoxedMinPerCell; --c) {
                const double share = std::min(1.0, (double)(1u << c) / std::max(per_row, 1.0));
                double cells = (share * R + R / coarse + 2.0) * (R / coarse + 2.0);
                if (D == 3) cells *= R / coarse + 2.0;
                if (cells * F * sizeof(float) <= 0.9 * (double)bp.budget) chunk_log2 = c;
            }
            if (chunk_log2 >= 0) {
                const uint32_t pieces = (uint32_t)std::min(64.0, std::ceil(per_row / (double)(1u << chunk_log2)) + 1.0);
                bp.tiled_level[bp.n_tiled] = (uint8_t)l;
                bp.tiled_chunk_log2[bp.n_tiled] = (uint8_t)chunk_log2;
                bp.tiled_pieces[bp.n_tiled] = (uint8_t)pieces;
                bp.tiled_start[bp.n_tiled + 1] = bp.tiled_start[bp.n_tiled] + bp.n_rows * pieces;
                ++bp.n_tiled;
                if (bp.budget > lds_bytes) lds_bytes = bp.budget;
            } else {
                bp.big_level[kept++] = (uint8_t)l;
            }
        }
        n_big = kept;
    }
    const unsigned long long blocks = (unsigned long long)bp.n_small * bp.small_blocks + bp.tiled_start[bp.n_tiled] + (unsigned long long)n_big * bp.big_blocks;
    if (blocks > 0x7fffffffull) return fail(TNN_ERR_UNSUPPORTED, "grid backward: batch too large for one launch");
    const dim3 grid((unsigned)blocks);
#define TNN_BWD(GT)                                                                                                    \
    do {                                                                                                               \
        auto k = grid_backward_kernel<D, F, GT, TAB>;                                                                  \
        if (lds_bytes > 48 * 1024 &&                                                                                   \
            hipFuncSetAttribute(reinterpret_cast<const void *>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess) \
            return fail(TNN_ERR_HIP, "cannot reserve %u bytes of LDS", lds_bytes);                                     \
        TNN_LAUNCH(k, grid, dim3(kBwdThreads), lds_bytes, s, lv, gp, bp, x, order, bin_start, (const GT *)dLdy, grad, (long long)M);    \
    } while (0)
    switch (dy_dtype) {
    case TNN_FP32: TNN_BWD(float); break;
    case TNN_BF16: TNN_BWD(bf16_t); break;
    case TNN_FP16: TNN_BWD(fp16_t); break;
    default: return fail(TNN_ERR_UNSUPPORTED, "dy_dtype %d", dy_dtype);
    }
#undef TNN_BWD
    return check_launch("grid_backward_kernel");
}

#define TNN_DISPATCH_DF(desc, CALL)                                                              \
    do {                                                                                         \
        const uint32_t F__ = (desc)->n_features_per_level;                                       \
        if ((desc)->n_dims == 2) {                                                               \
            constexpr int D_ = 2;                                                                \
            if (F__ == 1) { constexpr int F_ = 1; CALL; }                                        \
            else if (F__ == 2) { constexpr int F_ = 2; CALL; }                                   \
            else if (F__ == 4) { constexpr int F_ = 4; CALL; }                                   \
            else { constexpr int F_ = 8; CALL; }                                                 \
        } else {                                                                                 \
            constexpr int D_ = 3;                                                                \
            if (F__ == 1) { constexpr int F_ = 1; CALL; }                                        \
            else if (F__ == 2) { constexpr int F_ = 2; CALL; }                                   \
            else if (F__ == 4) { constexpr int F_ = 4; CALL; }                                   \
            else { constexpr int F_ = 8; CALL; }                                                 \
        }                                                                                        \
    } while (0)

} // namespace tnn

using namespace tnn;

TNN_API int tnn_grid_desc_init(tnn_grid_desc *desc, uint32_t n_dims, uint32_t n_levels, uint32_t n_features_per_level,
                               uint32_t log2_hashmap_size, uint32_t base_resolution, float per_level_scale,
                               uint32_t grid_type, uint32_t hash_type, uint32_t interpolation, uint32_t param_dtype) {
    if (!desc) return fail(TNN_ERR_INVALID_ARGUMENT, "desc is NULL");
    memset(desc, 0, sizeof(*desc));
    desc->n_dims = n_dims;
    desc->n_levels = n_levels;
    desc->n_features_per_level = n_features_per_level;
    desc->log2_hashmap_size = log2_hashmap_size;
    desc->base_resolution = base_resolution;
    desc->per_level_scale = per_level_scale;
    desc->grid_type = grid_type;
    desc->hash_type = hash_type;
    desc->interpolation = interpolation;
    desc->param_dtype = param_dtype;
    int rc = check_grid_desc(desc);
    if (rc) return rc;
    if (log2_hashmap_size > 31) return fail(TNN_ERR_INVALID_ARGUMENT, "log2_hashmap_size %u", log2_hashmap_size);
    if (base_resolution == 0 || !(per_level_scale > 0.0f)) return fail(TNN_ERR_INVALID_ARGUMENT, "base_resolution / per_level_scale");

    // include/encodings/grid.h:604-644 with grid_scale / grid_resolution (common_device.h:767-775)
    const float log2_pls = std::log2(per_level_scale);
    uint64_t offset = 0;
    for (uint32_t i = 0; i < n_levels; ++i) {
        const float scale = std::exp2((float)i * log2_pls) * (float)base_resolution - 1.0f;
        const uint32_t resolution = (uint32_t)std::ceil(scale) + 1u;
        const uint32_t max_params = UINT32_MAX / 2;
        uint32_t params_in_level;
        if (std::pow((float)resolution, (float)n_dims) > (float)max_params) {
            params_in_level = max_params;
        } else {
            params_in_level = 1;
            for (uint32_t k = 0; k < n_dims; ++k) params_in_level *= resolution;
        }
        params_in_level = (params_in_level + 7u) / 8u * 8u;
        if (grid_type == TNN_GRID_TILED) {
            uint32_t t = 1;
            for (uint32_t k = 0; k < n_dims; ++k) t *= base_resolution;
            if (t < params_in_level) params_in_level = t;
        } else if (grid_type == TNN_GRID_HASH) {
            const uint32_t t = 1u << log2_hashmap_size;
            if (t < params_in_level) params_in_level = t;
        }
        desc->offsets[i] = (uint32_t)offset;
        desc->scales[i] = scale;
        desc->resolutions[i] = resolution;
        offset += params_in_level;
        if (offset > UINT32_MAX) return fail(TNN_ERR_INVALID_ARGUMENT, "grid table exceeds 2^32 entries");
    }
    desc->offsets[n_levels] = (uint32_t)offset;
    return TNN_OK;
}

TNN_API size_t tnn_grid_n_params(const tnn_grid_desc *desc) {
    if (check_grid_desc(desc)) return 0;
    return (size_t)desc->offsets[desc->n_levels] * desc->n_features_per_level;
}

namespace tnn {
int grid_common(const tnn_grid_desc *desc, uint32_t padded_width, size_t M, GridLevels *lv, GridParams *gp) {
    int rc = check_grid_desc(desc);
    if (rc) return rc;
    // include/encodings/grid.h:665-677
    if (padded_width == 0) return fail(TNN_ERR_INVALID_ARGUMENT, "Can't have width == 0");
    if (padded_width < desc->n_levels * desc->n_features_per_level)
        return fail(TNN_ERR_INVALID_ARGUMENT, "Dimension mismatch grid encoding output: padded width %u < %u features", padded_width,
                    desc->n_levels * desc->n_features_per_level);
    if (M == 0) return fail(TNN_ERR_INVALID_ARGUMENT, "batch_size == 0");
    if (M > 0x7fffffffull * kGridThreads) return fail(TNN_ERR_INVALID_ARGUMENT, "batch too large");
    fill_levels(desc, lv);
    gp->n_levels = desc->n_levels;
    gp->hash_type = desc->hash_type;
    gp->interpolation = desc->interpolation;
    gp->padded_width = padded_width;
    return TNN_OK;
}
} // namespace tnn

TNN_API int tnn_grid_forward(const tnn_grid_desc *desc, const float *d_x, const void *d_table, void *d_out, int out_dtype,
                             uint32_t padded_width, size_t M, tnn_stream_t stream) {
    GridLevels lv;
    GridParams gp;
    int rc = grid_common(desc, padded_width, M, &lv, &gp);
    if (rc) return rc;
    if (!d_x || !d_table || !d_out) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    TNN_DISPATCH_DF(desc, rc = (launch_grid_forward_p<D_, F_>(desc, lv, gp, d_x, nullptr, d_table, d_out, out_dtype, M, as_stream(stream))));
    return rc;
}

TNN_API int tnn_grid_forward_ordered(const tnn_grid_desc *desc, const void *d_order, const void *d_table, void *d_out, int out_dtype,
                                     uint32_t padded_width, size_t M, tnn_stream_t stream) {
    GridLevels lv;
    GridParams gp;
    int rc = grid_common(desc, padded_width, M, &lv, &gp);
    if (rc) return rc;
    if (!d_order || !d_table || !d_out) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (reinterpret_cast<uintptr_t>(d_order) & 15) return fail(TNN_ERR_INVALID_ARGUMENT, "d_order must be 16-byte aligned");
    TNN_DISPATCH_DF(desc, rc = (launch_grid_forward_p<D_, F_>(desc, lv, gp, nullptr, static_cast<const float4 *>(d_order), d_table, d_out,
                                                              out_dtype, M, as_stream(stream))));
    return rc;
}

static int grid_backward_any(const tnn_grid_desc *desc, const float *d_x, const float4 *d_order, const void *d_dLdy, int dy_dtype,
                             uint32_t padded_width, void *d_grad_table, int grad_dtype, int overwrite, size_t M, tnn_stream_t stream) {
    GridLevels lv;
    GridParams gp;
    int rc = grid_common(desc, padded_width, M, &lv, &gp);
    if (rc) return rc;
    if ((!d_x && !d_order) || !d_dLdy || !d_grad_table) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (d_order && (reinterpret_cast<uintptr_t>(d_order) & 15)) return fail(TNN_ERR_INVALID_ARGUMENT, "d_order must be 16-byte aligned");
    if (grad_dtype != TNN_FP32 && grad_dtype != TNN_FP16) return fail(TNN_ERR_UNSUPPORTED, "gradient table dtype %d", grad_dtype);
    if (grad_dtype == TNN_FP16 && desc->n_features_per_level % 2 != 0)
        return fail(TNN_ERR_UNSUPPORTED, "fp16 gradient tables need an even number of features per level (features are added in pairs)");
    hipStream_t s = as_stream(stream);
    if (overwrite) {
        // a fill kernel rather than a memset node, so the call can be captured into a HIP graph
        const size_t bytes = tnn_grid_n_params(desc) * (grad_dtype == TNN_FP32 ? sizeof(float) : sizeof(fp16_t));
        if (reinterpret_cast<uintptr_t>(d_grad_table) & 15) return fail(TNN_ERR_INVALID_ARGUMENT, "d_grad_table must be 16-byte aligned");
        const size_t n4 = bytes / 16;
        const size_t n_tail = (bytes - n4 * 16) / sizeof(float); // level sizes are multiples of 8 entries: fp16 tables leave no tail
        size_t blocks = (n4 + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        if (blocks < 4) blocks = 4;
        TNN_LAUNCH(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (float4 *)d_grad_table, n4,
                   reinterpret_cast<float *>(static_cast<char *>(d_grad_table) + n4 * 16), n_tail);
        if ((rc = check_launch("fill_zero_kernel"))) return rc;
    }
    if (grad_dtype == TNN_FP32) {
        TNN_DISPATCH_DF(desc, rc = (launch_grid_backward_g<D_, F_, float>(lv, gp, d_x, d_order, d_dLdy, dy_dtype, (float *)d_grad_table, M, s)));
    } else {
        const uint32_t F = desc->n_features_per_level;
#define TNN_PACKED(D_, F_) rc = launch_grid_backward_g<D_, F_, fp16_t>(lv, gp, d_x, d_order, d_dLdy, dy_dtype, (fp16_t *)d_grad_table, M, s)
        if (desc->n_dims == 2) {
            if (F == 2) TNN_PACKED(2, 2); else if (F == 4) TNN_PACKED(2, 4); else TNN_PACKED(2, 8);
        } else {
            if (F == 2) TNN_PACKED(3, 2); else if (F == 4) TNN_PACKED(3, 4); else TNN_PACKED(3, 8);
        }
#undef TNN_PACKED
    }
    return rc;
}

TNN_API int tnn_grid_backward(const tnn_grid_desc *desc, const float *d_x, const void *d_dLdy, int dy_dtype,
                              uint32_t padded_width, float *d_grad_table, int overwrite, size_t M, tnn_stream_t stream) {
    return grid_backward_any(desc, d_x, nullptr, d_dLdy, dy_dtype, padded_width, d_grad_table, TNN_FP32, overwrite, M, stream);
}

TNN_API int tnn_grid_backward_ordered(const tnn_grid_desc *desc, const void *d_order, const void *d_dLdy, int dy_dtype,
                                      uint32_t padded_width, float *d_grad_table, int overwrite, size_t M, tnn_stream_t stream) {
    if (!d_order) return tnn::fail(TNN_ERR_INVALID_ARGUMENT, "d_order is NULL");
    return grid_backward_any(desc, nullptr, static_cast<const float4 *>(d_order), d_dLdy, dy_dtype, padded_width, d_grad_table, TNN_FP32, overwrite,
                             M, stream);
}

TNN_API int tnn_grid_backward_packed(const tnn_grid_desc *desc, const float *d_x, const void *d_dLdy, int dy_dtype,
                                     uint32_t padded_width, void *d_grad_table_f16, int overwrite, size_t M, tnn_stream_t stream) {
    return grid_backward_any(desc, d_x, nullptr, d_dLdy, dy_dtype, padded_width, d_grad_table_f16, TNN_FP16, overwrite, M, stream);
}

TNN_API int tnn_grid_indices(const tnn_grid_desc *desc, const float *d_x, uint32_t *d_indices, size_t M, tnn_stream_t stream) {
    GridLevels lv;
    GridParams gp;
    int rc = grid_common(desc, desc ? desc->n_levels * desc->n_features_per_level : 0, M, &lv, &gp);
    if (rc) return rc;
    if (!d_x || !d_indices) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    const unsigned blocks = (unsigned)((M + kGridThreads - 1) / kGridThreads);
    if (desc->n_dims == 2)
        TNN_LAUNCH((grid_indices_kernel<2>), dim3(blocks), dim3(kGridThreads), 0, as_stream(stream), lv, gp, d_x, d_indices, (long long)M);
    else
        TNN_LAUNCH((grid_indices_kernel<3>), dim3(blocks), dim3(kGridThreads), 0, as_stream(stream), lv, gp, d_x, d_indices, (long long)M);
    return check_launch("grid_indices_kernel");
}
