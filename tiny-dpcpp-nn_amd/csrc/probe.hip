// Measurement aid: what the memory system delivers for the access pattern that bounds the hash-grid gather, with nothing
// else in the kernel. Every thread stands for one point of a batch and reads 4 bytes from each of `lines_per_thread` lines of
// 128 bytes chosen at random in a buffer, all of them in flight at once in groups of 32 (as the encoding kernel has the
// 4 levels x 8 corners of a group in flight), and keeps the sum. No two lanes share a line except by chance: the situation
// of the finest levels of a table, whose cells are fewer than the points. No counterpart in the reference.
#include "tnn_internal.h"

namespace tnn {

constexpr int kProbeThreads = 256; // the workgroup size of the encoding kernel

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) { // (lowbias32, Wellons)
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

__global__ void __launch_bounds__(kProbeThreads)
    line_gather_probe_kernel(const uint32_t *__restrict__ buf, uint32_t n_lines, int groups, uint32_t seed, uint32_t *__restrict__ sink, long long n) {
    const long long tid = (long long)blockIdx.x * kProbeThreads + threadIdx.x;
    if (tid >= n) return;
    uint32_t acc = 0;
    for (int g = 0; g < groups; ++g) {
        uint32_t v[32];
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            const uint32_t line = probe_hash((uint32_t)tid * 2654435761u + (uint32_t)(g * 32 + k) * 40503u + seed) % n_lines;
            v[k] = buf[(size_t)line * 32 + (threadIdx.x & 31)];
        }
#pragma unroll
        for (int k = 0; k < 32; ++k) acc += v[k];
    }
    sink[tid] = acc;
}

} // namespace tnn

using namespace tnn;

TNN_API int tnn_probe_line_gather(const void *d_buffer, size_t buffer_bytes, size_t n_threads, int lines_per_thread, uint32_t seed, void *d_sink,
                                  tnn_stream_t stream) {
    if (!d_buffer || !d_sink) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (buffer_bytes < 128 || (buffer_bytes >> 7) > 0xFFFFFFFFull) return fail(TNN_ERR_INVALID_ARGUMENT, "buffer of %zu bytes", buffer_bytes);
    if (n_threads == 0 || lines_per_thread < 32 || lines_per_thread % 32 != 0)
        return fail(TNN_ERR_INVALID_ARGUMENT, "lines_per_thread must be a positive multiple of 32 and n_threads positive");
    const size_t blocks = (n_threads + kProbeThreads - 1) / kProbeThreads;
    if (blocks > 0x7FFFFFFFull) return fail(TNN_ERR_INVALID_ARGUMENT, "too many threads");
    TNN_LAUNCH(line_gather_probe_kernel, dim3((unsigned)blocks), dim3(kProbeThreads), 0, as_stream(stream), (const uint32_t *)d_buffer,
               (uint32_t)(buffer_bytes >> 7), lines_per_thread / 32, seed, (uint32_t *)d_sink, (long long)n_threads);
    return check_launch("line_gather_probe_kernel");
}
