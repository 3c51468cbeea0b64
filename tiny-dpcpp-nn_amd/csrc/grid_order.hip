// Cell order for the points of a batch (gfx950): a permutation of the rows that puts points of the same part of space
// next to each other, so that the lanes of a wave and the waves of a workgroup gather from the same 128-byte lines of
// the grid's table at the same time. A random batch misses L2 on almost every gather of a level beyond 4 MiB and pays
// a whole line per 4-byte entry; in cell order the dense and the coarser hashed levels share their lines. Every row's
// result is computed exactly as before, in another lane, and written to its own row: results do not change.
//
// The reference has no such pass: its kernel_grid (include/encodings/grid.h:37-135) takes the points as they come, one
// work-item per (point, level), levels as the slow grid dimension (:696-731).
//
// Two steps, neither needs a stable order:
//   1. counting sort by a 12-bit key, the leading bits of every coordinate with the first dimension fastest (x runs along
//      a table line): per-workgroup histograms in LDS, one small scan kernel, scatter with LDS counters;
//   2. inside every one of the 4096 bins, a counting sort in LDS by the next bits of every coordinate.
// A record is 16 bytes: up to three coordinates and the row number.
#include "grid_device.h"

namespace tnn {

constexpr int kOrderThreads = 1024;
constexpr int kOrderBins = 4096;      // 12-bit key
constexpr int kOrderGroups = 64;      // runs of 64 bins, one scan workgroup each
constexpr int kOrderMaxWg = 256;      // histogram workgroups (the scan keeps a [workgroups][64] tile in LDS)
constexpr int kRefineCap = 2048;      // records of a bin sorted in LDS at once (32 KiB)
constexpr int kRefineThreads = 256;
constexpr int kRefineBins = 64;       // 6 further bits

struct OrderPlan {
    int n_wg;
    long long chunk; // points per histogram workgroup, a multiple of kOrderThreads
    size_t record_bytes, hist_bytes, group_bytes;
};

static OrderPlan order_plan(size_t M) {
    OrderPlan p;
    long long wg = ((long long)M + 4 * kOrderThreads - 1) / (4 * kOrderThreads); // at least four rounds per workgroup
    if (wg > kOrderMaxWg) wg = kOrderMaxWg;
    if (wg < 1) wg = 1;
    p.n_wg = (int)wg;
    long long chunk = ((long long)M + wg - 1) / wg;
    p.chunk = (chunk + kOrderThreads - 1) / kOrderThreads * kOrderThreads;
    p.record_bytes = order_record_bytes(M);
    p.hist_bytes = (size_t)p.n_wg * kOrderBins * sizeof(uint32_t);
    p.group_bytes = (size_t)p.n_wg * kOrderGroups * sizeof(uint32_t);
    return p;
}

// Leading `bits` bits of a coordinate taken as a number in [0, 1); anything else (outside, NaN) goes to an end bin.
__device__ __forceinline__ uint32_t quantise(float v, int bits) {
    const float s = v * (float)(1 << bits);
    if (!(s > 0.0f)) return 0;
    const uint32_t q = (uint32_t)s;
    return q < (1u << bits) ? q : (1u << bits) - 1;
}

template <int D> struct OrderBits;
template <> struct OrderBits<2> { static constexpr int coarse = 6, fine = 3; };
template <> struct OrderBits<3> { static constexpr int coarse = 4, fine = 2; };

template <int D> __device__ __forceinline__ uint32_t coarse_key(const float (&x)[D]) {
    constexpr int b = OrderBits<D>::coarse;
    uint32_t k = 0;
#pragma unroll
    for (int d = 0; d < D; ++d) k |= quantise(x[d], b) << (b * d);
    return k;
}
template <int D> __device__ __forceinline__ uint32_t fine_key(const float (&x)[D]) {
    constexpr int b = OrderBits<D>::coarse, f = OrderBits<D>::fine;
    uint32_t k = 0;
#pragma unroll
    for (int d = 0; d < D; ++d) k |= (quantise(x[d], b + f) & ((1u << f) - 1)) << (f * d);
    return k;
}

template <int D> __device__ __forceinline__ void load_point(const float *__restrict__ xin, long long i, float (&x)[D]) {
#pragma unroll
    for (int d = 0; d < D; ++d) x[d] = xin[i * D + d];
}

// Step 1a: histogram of the workgroup's chunk of points over the 4096 bins, and its totals per run of 64 bins.
template <int D>
__global__ void __launch_bounds__(kOrderThreads)
    order_hist_kernel(const float *__restrict__ xin, long long M, long long chunk, uint32_t *__restrict__ hist, uint32_t *__restrict__ group_totals) {
    __shared__ uint32_t h[kOrderBins];
    for (int b = threadIdx.x; b < kOrderBins; b += kOrderThreads) h[b] = 0;
    __syncthreads();
    const long long begin = (long long)blockIdx.x * chunk;
    long long end = begin + chunk;
    if (end > M) end = M;
    for (long long i = begin + threadIdx.x; i < end; i += kOrderThreads) {
        float x[D];
        load_point<D>(xin, i, x);
        atomicAdd(&h[coarse_key<D>(x)], 1u);
    }
    __syncthreads();
    uint32_t *mine = hist + (size_t)blockIdx.x * kOrderBins;
    for (int b = threadIdx.x; b < kOrderBins; b += kOrderThreads) mine[b] = h[b];
    if (threadIdx.x < kOrderGroups) {
        uint32_t s = 0;
        for (int i = 0; i < 64; ++i) s += h[64 * threadIdx.x + ((i + threadIdx.x) & 63)]; // skewed: no two lanes on one bank
        group_totals[(size_t)blockIdx.x * kOrderGroups + threadIdx.x] = s;
    }
}

// Step 1b: turns the histograms into starting positions, in place. Bins are laid out in key order, and inside a bin the
// workgroups in their own order. Workgroup g of this kernel owns bins [64 g, 64 g + 64). The prefix over the workgroups of
// a bin is a chain of dependent LDS accesses, so the sixteen waves each take a sixteenth of the workgroups (lane = bin)
// and the sixteen partial sums per bin are put together afterwards.
constexpr int kScanThreads = 1024;
constexpr int kScanParts = kScanThreads / 64;
__global__ void __launch_bounds__(kScanThreads)
    order_scan_kernel(uint32_t *__restrict__ hist, const uint32_t *__restrict__ group_totals, int n_wg) {
    extern __shared__ uint32_t tile[]; // [n_wg][64] counts, then [parts][64] partial sums, then 64 bin starts, then the wave sums
    uint32_t *part_sum = tile + (size_t)n_wg * 64;
    uint32_t *bin_start = part_sum + kScanParts * 64;
    uint32_t *wave_sum = bin_start + 64;
    const int g = blockIdx.x, tid = threadIdx.x, bin = tid & 63, part = tid >> 6;
    // everything in front of this run of bins
    uint32_t before = 0;
    for (int e = tid; e < n_wg * kOrderGroups; e += kScanThreads) // coalesced, every load independent of the one before
        before += ((e & (kOrderGroups - 1)) < g) ? group_totals[e] : 0u;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) before += __shfl_down(before, off, 64);
    if (bin == 0) wave_sum[part] = before;
    for (int e = tid; e < n_wg * 64; e += kScanThreads) tile[e] = hist[(size_t)(e >> 6) * kOrderBins + 64 * g + (e & 63)];
    __syncthreads();
    // exclusive prefix over this wave's workgroups of one bin (lanes on consecutive words: no bank conflicts)
    const int per = (n_wg + kScanParts - 1) / kScanParts;
    const int w_begin = part * per, w_end = (w_begin + per < n_wg) ? w_begin + per : n_wg;
    uint32_t run = 0;
    for (int w = w_begin; w < w_end; ++w) {
        const uint32_t c = tile[w * 64 + bin];
        tile[w * 64 + bin] = run;
        run += c;
    }
    part_sum[part * 64 + bin] = run;
    __syncthreads();
    if (tid < 64) {
        uint32_t base = 0;
#pragma unroll
        for (int i = 0; i < kScanParts; ++i) base += wave_sum[i];
        // the parts of a bin one after the other, then an exclusive prefix over the 64 bins
        uint32_t total = 0;
#pragma unroll
        for (int i = 0; i < kScanParts; ++i) {
            const uint32_t c = part_sum[i * 64 + tid];
            part_sum[i * 64 + tid] = total;
            total += c;
        }
        uint32_t incl = total;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t v = __shfl_up(incl, off, 64);
            if (tid >= off) incl += v;
        }
        bin_start[tid] = base + incl - total;
    }
    __syncthreads();
    for (int e = tid; e < n_wg * 64; e += kScanThreads)
        hist[(size_t)(e >> 6) * kOrderBins + 64 * g + (e & 63)] = tile[e] + part_sum[((e >> 6) / per) * 64 + (e & 63)] + bin_start[e & 63];
}

// Step 1c: every point goes to the next free position of its bin (the workgroup's own counters, in LDS).
template <int D>
__global__ void __launch_bounds__(kOrderThreads)
    order_scatter_kernel(const float *__restrict__ xin, long long M, long long chunk, const uint32_t *__restrict__ starts, float4 *__restrict__ records) {
    __shared__ uint32_t next[kOrderBins];
    const uint32_t *mine = starts + (size_t)blockIdx.x * kOrderBins;
    for (int b = threadIdx.x; b < kOrderBins; b += kOrderThreads) next[b] = mine[b];
    __syncthreads();
    const long long begin = (long long)blockIdx.x * chunk;
    long long end = begin + chunk;
    if (end > M) end = M;
    for (long long i = begin + threadIdx.x; i < end; i += kOrderThreads) {
        float x[D];
        load_point<D>(xin, i, x);
        const uint32_t pos = atomicAdd(&next[coarse_key<D>(x)], 1u);
        float4 r;
        r.x = x[0];
        r.y = x[1];
        r.z = (D > 2) ? x[D - 1] : 0.0f;
        r.w = __uint_as_float((uint32_t)i);
        records[pos] = r;
    }
}

// Step 2: one workgroup per bin sorts the bin's records by the next bits of the coordinates, in LDS, in pieces of at most
// kRefineCap records (a bin that holds more, because the points cluster, is refined piece by piece).
template <int D>
__global__ void __launch_bounds__(kRefineThreads)
    order_refine_kernel(const uint32_t *__restrict__ starts, float4 *__restrict__ records, long long M) {
    __shared__ float4 rec[kRefineCap];
    __shared__ uint32_t count[kRefineBins], next[kRefineBins];
    const int bin = blockIdx.x, tid = threadIdx.x;
    const long long begin = starts[bin]; // workgroup 0's start of a bin is the start of the bin
    const long long end = (bin + 1 < kOrderBins) ? (long long)starts[bin + 1] : M;
    for (long long p0 = begin; p0 < end; p0 += kRefineCap) {
        const int n = (int)((end - p0 < kRefineCap) ? end - p0 : kRefineCap);
        if (tid < kRefineBins) count[tid] = 0;
        __syncthreads();
        uint32_t key[kRefineCap / kRefineThreads];
#pragma unroll
        for (int u = 0; u < kRefineCap / kRefineThreads; ++u) {
            const int e = tid + u * kRefineThreads;
            key[u] = 0;
            if (e < n) {
                const float4 r = records[p0 + e];
                rec[e] = r;
                float x[D];
                x[0] = r.x;
                x[1] = r.y;
                if (D > 2) x[D - 1] = r.z;
                key[u] = fine_key<D>(x);
                atomicAdd(&count[key[u]], 1u);
            }
        }
        __syncthreads();
        if (tid < kRefineBins) {
            const uint32_t c = count[tid];
            uint32_t incl = c;
#pragma unroll
            for (int off = 1; off < kRefineBins; off <<= 1) {
                const uint32_t v = __shfl_up(incl, off, 64);
                if (tid >= off) incl += v;
            }
            next[tid] = incl - c;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kRefineCap / kRefineThreads; ++u) {
            const int e = tid + u * kRefineThreads;
            if (e < n) records[p0 + atomicAdd(&next[key[u]], 1u)] = rec[e];
        }
        __syncthreads();
    }
}

} // namespace tnn

using namespace tnn;

TNN_API size_t tnn_grid_order_bytes(const tnn_grid_desc *desc, size_t M) {
    if (check_grid_desc(desc) || M == 0) return 0;
    const OrderPlan p = order_plan(M);
    return p.record_bytes + p.hist_bytes + p.group_bytes + 256;
}

TNN_API int tnn_grid_order_points(const tnn_grid_desc *desc, const float *d_x, size_t M, void *d_order, size_t order_bytes,
                                  tnn_stream_t stream) {
    int rc = check_grid_desc(desc);
    if (rc) return rc;
    if (!d_x || !d_order) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (M == 0) return fail(TNN_ERR_INVALID_ARGUMENT, "batch_size == 0");
    if (M > 0xffffffffull) return fail(TNN_ERR_INVALID_ARGUMENT, "row numbers are 32 bits: at most 2^32 - 1 points");
    if (reinterpret_cast<uintptr_t>(d_order) & 255) return fail(TNN_ERR_INVALID_ARGUMENT, "d_order must be 256-byte aligned");
    const size_t need = tnn_grid_order_bytes(desc, M);
    if (order_bytes < need) return fail(TNN_ERR_WORKSPACE, "order buffer of %zu bytes given, %zu needed", order_bytes, need);
    const OrderPlan p = order_plan(M);
    float4 *records = static_cast<float4 *>(d_order);
    uint32_t *hist = reinterpret_cast<uint32_t *>(static_cast<char *>(d_order) + p.record_bytes);
    uint32_t *groups = reinterpret_cast<uint32_t *>(static_cast<char *>(d_order) + p.record_bytes + p.hist_bytes);
    hipStream_t s = as_stream(stream);
    const size_t scan_lds = ((size_t)p.n_wg * 64 + kScanParts * 64 + 64 + kScanParts) * sizeof(uint32_t);
    if (scan_lds > 48 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void *>(order_scan_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)scan_lds) != hipSuccess)
        return fail(TNN_ERR_HIP, "cannot reserve %zu bytes of LDS", scan_lds);
#define TNN_ORDER(D_)                                                                                                                  \
    do {                                                                                                                               \
        TNN_LAUNCH((order_hist_kernel<D_>), dim3(p.n_wg), dim3(kOrderThreads), 0, s, d_x, (long long)M, p.chunk, hist, groups);         \
        if ((rc = check_launch("order_hist_kernel"))) return rc;                                                                       \
        TNN_LAUNCH(order_scan_kernel, dim3(kOrderGroups), dim3(kScanThreads), scan_lds, s, hist, (const uint32_t *)groups, p.n_wg);              \
        if ((rc = check_launch("order_scan_kernel"))) return rc;                                                                       \
        TNN_LAUNCH((order_scatter_kernel<D_>), dim3(p.n_wg), dim3(kOrderThreads), 0, s, d_x, (long long)M, p.chunk, (const uint32_t *)hist, records); \
        if ((rc = check_launch("order_scatter_kernel"))) return rc;                                                                    \
        TNN_LAUNCH((order_refine_kernel<D_>), dim3(kOrderBins), dim3(kRefineThreads), 0, s, (const uint32_t *)hist, records, (long long)M); \
        return check_launch("order_refine_kernel");                                                                                    \
    } while (0)
    if (desc->n_dims == 2) TNN_ORDER(2);
    TNN_ORDER(3);
#undef TNN_ORDER
}
