// Fully fused MLP for gfx950: inference, training forward, fused backward (delta propagation),
// weight gradients. One wave streams a tile of 32 batch rows through every layer:
//   * the transposed product  Y^T = W^T * X^T  is evaluated with v_mfma_f32_32x32x16_{bf16,f16}:
//     the weights are the A operand (staged once per workgroup in LDS, already in operand order),
//     the activations are the B operand and never leave the registers between layers;
//   * lane (j = lane % 32, h = lane / 32) owns batch row j of the tile; for every block of 16
//     features it holds the 8 features 16*kb + 8*h + [0, 8), i.e. one aligned 16-byte piece of the
//     row-major row. Loads, stores and MFMA B operands all use that same register layout.
//
// Reference behaviour being reproduced: include/network/kernel_esimd.h:565-640 (forward /
// inference), :160-228 (delta propagation), :230-239 (dW = delta^T * a), rounding points
// :443-487 (fp32 accumulate -> round to T -> activation; backward mask / sigmoid slope applied to
// the fp32 accumulator before rounding).
#include "mlp_tile.h"
#include "mlp_train_shape.h"
#include "mlp_backward128.inc"

#include <cstdlib>

namespace tnn {

// ------------------------------------------------------------------------------------------
// Operand preparation
// ------------------------------------------------------------------------------------------

// Operand order ("prepared" layout), per weight matrix l, per 32-row output tile a, per 16-deep
// contraction block kb: 64 lanes x 8 elements, lane = 32*h + i, element t:
//   forward : W_l[k = 16*kb + 8*h + t][n = 32*a + swap23(i)]
//   backward: W_l[k = 32*a + swap23(i)][n = 16*kb + 8*h + t]      (the product with W_l^T)
// Rows beyond the width (only for width 16, whose single tile is half empty) are zero.
template <typename T, typename SRC>
__global__ void prepare_weights_kernel(const SRC *__restrict__ packed, T *__restrict__ fwd, T *__restrict__ bwd, int W,
                                       int n_mats) {
    const int NI = (W + 31) / 32, NK = W / 16;
    const int per_mat = NI * NK * 512;
    const int total = n_mats * per_mat;
    for (int idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        const int l = idx / per_mat;
        int r = idx % per_mat;
        const int t = r & 7;
        const int lane = (r >> 3) & 63;
        r >>= 9;
        const int kb = r % NK, a = r / NK;
        const int h = lane >> 5, i = lane & 31;
        const int outer = 32 * a + swap23(i);  // output feature of the product
        const int inner = 16 * kb + 8 * h + t; // contraction index
        const SRC *src = packed + (size_t)l * W * W;
        T vf = (T)0.0f, vb = (T)0.0f;
        if (outer < W) {
            vf = (T)(float)src[packed_coord(inner, outer, W)]; // W[k = inner][n = outer]
            vb = (T)(float)src[packed_coord(outer, inner, W)]; // W[k = outer][n = inner]
        }
        if (fwd) fwd[idx] = vf;
        if (bwd) bwd[idx] = vb;
    }
}

// ------------------------------------------------------------------------------------------
// Forward / inference
// ------------------------------------------------------------------------------------------
// out: STORE_INTERM ? (n_mats + 1) matrices M x W ([0] = copy of x) : one matrix M x W.
// ACT (hidden activation) is a compile-time constant so that the layer loop stays one basic block:
// the fragments of the next matrix are requested from LDS before the current accumulators are
// converted, and arrive while the conversion runs.
// STAGED: every wave has a tile of LDS behind the weights and writes its rows through it (Tile::store_staged);
// 2 = with the streaming hint.
template <typename T, int W, int ACT, bool STORE_INTERM, bool W_IN_LDS, int THREADS, int STAGED = 0>
__global__ void __launch_bounds__(THREADS, (THREADS >= 512 && W <= 64) ? 4 : 1)
    mlp_forward_kernel(const typename Storage<T>::vec8 *__restrict__ wprep, const T *__restrict__ x, T *__restrict__ out,
                       int n_mats, int out_act, long long M) {
    typedef Tile<T, W> TL;
    typedef typename Storage<T>::vec8 vec8;
    constexpr int NK = TL::NK, NI = TL::NI;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    vec8 *lds_w = reinterpret_cast<vec8 *>(smem_raw);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 31, h = lane >> 5;
    const long long n_tiles = (M + 31) / 32;
    const long long stride = (long long)gridDim.x * (blockDim.x >> 6);
    long long tile = (long long)blockIdx.x * (blockDim.x >> 6) + wave;
    unsigned char *my_stage = smem_raw + (size_t)n_mats * (TL::NF * kWaveSize * sizeof(vec8)) + (size_t)wave * TL::TILE_BYTES;
    unsigned int st_off[NK];
    auto put = [&](const vec8(&r)[NK], T *dst, long long row, bool valid) __attribute__((always_inline)) {
        if constexpr (STAGED != 0) {
            TL::stage(r, my_stage, j, h);
            TL::template store_staged<(STAGED == 2 ? kStreamingStore : 0)>(my_stage, lane, TL::rows_of(dst, M), st_off);
        } else {
            TL::store(r, dst, row, h, valid);
        }
    };

    vec8 cur[NK];
    if constexpr (W_IN_LDS) {
        // The weights are requested first and the first tile behind them: the wait for the weights then leaves the tile's
        // loads in flight, and the workgroup passes its barrier as soon as the weights are there. Every other wave asks
        // for its first tile only behind that barrier, so that the workgroup's waves do not all wait for rows, compute and
        // store in the same phase (measured at width 64 with 5 matrices: 8.8 -> 7.8 us at 2^17 rows, where a wave has one
        // tile and nothing else overlaps its loads; 1-4 % at 2^18 and 2^20 rows).
        constexpr int per_mat = NI * NK * kWaveSize;
        const int n = n_mats * per_mat;
        constexpr int HELD = 4;
        vec8 held[HELD];
#pragma unroll
        for (int i = 0; i < HELD; ++i) {
            const int f = threadIdx.x + i * THREADS;
            held[i] = wprep[f < n ? f : n - 1];
        }
        asm volatile("" ::: "memory");
        const bool early = (wave & 1) == 0;
        if (early && tile < n_tiles) TL::load(cur, x, tile * 32 + j, h, tile * 32 + j < M);
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < HELD; ++i) {
            const int f = threadIdx.x + i * THREADS;
            if (f < n) lds_w[f] = held[i];
        }
        for (int f = threadIdx.x + HELD * THREADS; f < n; f += THREADS) lds_w[f] = wprep[f];
        __syncthreads();
        if (!early && tile < n_tiles) TL::load(cur, x, tile * 32 + j, h, tile * 32 + j < M);
    } else {
        if (tile < n_tiles) TL::load(cur, x, tile * 32 + j, h, tile * 32 + j < M);
    }
    // Where a tile is waited for. The hardware counts outstanding memory operations in order, and the compiler, which
    // places the waits, only knows an upper bound per register at a loop header: left to itself it waits for `cur` inside
    // the layer loop with a count of 0, i.e. also for the next tile's loads that were issued a moment before, and no
    // tile is ever computed while the next one is on its way. Passing `cur` through an empty asm statement pins the wait
    // to that place: here, where nothing younger is in flight, and below right after the copy from `nxt`, before the
    // tile's stores are issued. Inside the loop `cur` then never depends on memory.
    auto settle = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < NK; ++kb) asm volatile("" : "+v"(cur[kb]));
    };
    settle();

    while (tile < n_tiles) {
        const long long row = tile * 32 + j;
        const bool valid = row < M;
        // prefetch the next tile of this wave while the current one is being computed
        const long long next_tile = tile + stride;
        vec8 nxt[NK];
        if (next_tile < n_tiles) TL::load(nxt, x, next_tile * 32 + j, h, next_tile * 32 + j < M);

        if constexpr (STAGED != 0) TL::row_offsets(st_off, tile, lane, M);
        if (STORE_INTERM) put(cur, out, row, valid);
        f32x16 acc[NI];
        for (int l = 0; l < n_mats - 1; ++l) {
            TL::template matmul<W_IN_LDS>(acc, cur, lds_w, wprep, l, lane);
            TL::template repack<ACT>(cur, acc);
            if (STORE_INTERM) put(cur, out + (size_t)(l + 1) * M * W, row, valid);
        }
        TL::template matmul<W_IN_LDS>(acc, cur, lds_w, wprep, n_mats - 1, lane);
        vec8 res[NK];
        TL::repack_rt(res, acc, out_act);
        if (!STORE_INTERM && next_tile < n_tiles) {
            // inference: take the next tile over before this one's stores go out (waiting afterwards would wait for them too)
#pragma unroll
            for (int kb = 0; kb < NK; ++kb) cur[kb] = nxt[kb];
            settle();
        }
        put(res, STORE_INTERM ? out + (size_t)n_mats * M * W : out, row, valid);
        if (STORE_INTERM && next_tile < n_tiles) {
#pragma unroll
            for (int kb = 0; kb < NK; ++kb) cur[kb] = nxt[kb];
            settle();
        }
        tile = next_tile;
    }
}

// ------------------------------------------------------------------------------------------
// Forward for networks whose weights do not fit LDS (width 128 with more than four matrices): the
// matrices stream through a double-buffered LDS slot, one layer at a time, for a round of 512 batch
// rows (8 waves x 2 tiles of 32 rows). While a layer is being computed from one slot, every thread
// carries its 64-byte share of the next matrix from L2 to the other slot; one barrier per layer. A
// wave feeds each weight fragment it reads from LDS to two MFMAs (its two tiles), which halves the
// LDS traffic per flop; reading the fragments from global memory instead (as the in-LDS kernel
// does when it has no room) is bound by the vector cache at 16 % of the MFMA peak.
// ------------------------------------------------------------------------------------------
constexpr int kStreamThreads = 512;
constexpr int kStreamTiles = 2;

// STAGED as in mlp_forward_kernel: 0 plain stores, 1 whole rows through a tile of LDS per wave (behind the two slots),
// 2 the same with the streaming hint.
template <typename T, int W, int ACT, bool STORE_INTERM, int STAGED = 0>
__global__ void __launch_bounds__(kStreamThreads, 1)
    mlp_forward_stream_kernel(const typename Storage<T>::vec8 *__restrict__ wprep, const T *__restrict__ x, T *__restrict__ out,
                              int n_mats, int out_act, long long M, int store_input) {
    typedef Tile<T, W> TL;
    typedef typename Storage<T>::vec8 vec8;
    constexpr int NK = TL::NK, NI = TL::NI, R = kStreamTiles;
    constexpr int per_mat = NI * NK * kWaveSize;         // 16-byte fragments per matrix
    constexpr int SHARE = per_mat / kStreamThreads;      // fragments a thread carries per matrix
    static_assert(per_mat % kStreamThreads == 0, "matrix does not split evenly over the workgroup");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    vec8 *lds = reinterpret_cast<vec8 *>(smem_raw); // slot s starts at lds + s * per_mat

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 31, h = lane >> 5;
    constexpr int ROUND = (kStreamThreads / 64) * R * 32;
    const long long n_rounds = (M + ROUND - 1) / ROUND;

    vec8 st[SHARE];
#pragma unroll
    for (int i = 0; i < SHARE; ++i) lds[threadIdx.x + kStreamThreads * i] = wprep[threadIdx.x + kStreamThreads * i];
    int b = 0; // slot that holds the matrix of the layer about to run
    unsigned char *my_stage = smem_raw + 2 * per_mat * sizeof(vec8) + (size_t)wave * TL::TILE_BYTES;

    for (long long r = blockIdx.x; r < n_rounds; r += gridDim.x) {
        long long row[R];
        bool valid[R];
        vec8 cur[R][NK];
        unsigned int st_base[R];
        auto put = [&](int t, T *dst) __attribute__((always_inline)) {
            if constexpr (STAGED != 0) {
                TL::stage(cur[t], my_stage, j, h);
                TL::template store_staged_at<(STAGED == 2 ? kStreamingStore : 0)>(my_stage, lane, TL::rows_of(dst, M), st_base[t]);
            } else {
                TL::store(cur[t], dst, row[t], h, valid[t]);
            }
        };
#pragma unroll
        for (int t = 0; t < R; ++t) {
            row[t] = r * ROUND + (wave * R + t) * 32 + j;
            valid[t] = row[t] < M;
            if constexpr (STAGED != 0) st_base[t] = TL::staged_base(r * (ROUND / 32) + wave * R + t, lane);
            TL::load(cur[t], x, row[t], h, valid[t]);
            if (STORE_INTERM && store_input) put(t, out); // (a training step reads the input where it is: it leaves matrix 0 unwritten)
        }
        const bool more_rounds = r + gridDim.x < n_rounds;
        for (int l = 0; l < n_mats; ++l) {
            __syncthreads(); // the matrix of layer l is in slot b; nobody reads the other slot any more
            const bool last = l + 1 == n_mats;
            const bool stage = !last || more_rounds;
            const vec8 *next = wprep + (size_t)(last ? 0 : l + 1) * per_mat;
            if (stage) {
#pragma unroll
                for (int i = 0; i < SHARE; ++i) st[i] = next[threadIdx.x + kStreamThreads * i];
            }
            f32x16 acc[R][NI];
#pragma unroll
            for (int t = 0; t < R; ++t)
#pragma unroll
                for (int a = 0; a < NI; ++a) acc[t][a] = f32x16{};
            const vec8 *w = lds + b * per_mat + lane;
#pragma unroll
            for (int kb = 0; kb < NK; ++kb) {
#pragma unroll
                for (int a = 0; a < NI; ++a) {
                    const vec8 frag = w[(a * NK + kb) * kWaveSize];
#pragma unroll
                    for (int t = 0; t < R; ++t) acc[t][a] = Storage<T>::mfma(frag, cur[t][kb], acc[t][a]);
                }
            }
            if (stage) {
#pragma unroll
                for (int i = 0; i < SHARE; ++i) lds[(b ^ 1) * per_mat + threadIdx.x + kStreamThreads * i] = st[i];
            }
#pragma unroll
            for (int t = 0; t < R; ++t) {
                if (!last) {
                    TL::template repack<ACT>(cur[t], acc[t]);
                    if (STORE_INTERM) put(t, out + (size_t)(l + 1) * M * W);
                } else {
                    TL::repack_rt(cur[t], acc[t], out_act);
                    put(t, STORE_INTERM ? out + (size_t)n_mats * M * W : out);
                }
            }
            b ^= 1;
        }
    }
}

// ------------------------------------------------------------------------------------------
// Backward: delta propagation (include/network/kernel_esimd.h:186-227)
// ------------------------------------------------------------------------------------------
template <typename T, int W, bool W_IN_LDS>
__global__ void __launch_bounds__(kFwdThreads)
    mlp_backward_kernel(const typename Storage<T>::vec8 *__restrict__ wprep_bwd, const T *__restrict__ dLdy,
                        const T *__restrict__ interm_fwd, T *__restrict__ interm_bwd, T *__restrict__ dLdx, int n_mats,
                        int act, int out_act, long long M) {
    typedef Tile<T, W> TL;
    typedef typename Storage<T>::vec8 vec8;
    constexpr int NK = TL::NK, NI = TL::NI;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    vec8 *lds_w = reinterpret_cast<vec8 *>(smem_raw);
    if (W_IN_LDS) stage_weights<T, W>(lds_w, wprep_bwd, n_mats);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 31, h = lane >> 5;
    const long long n_tiles = (M + 31) / 32;
    const long long stride = (long long)gridDim.x * (blockDim.x >> 6);
    const size_t mat = (size_t)M * W;

    for (long long tile = (long long)blockIdx.x * (blockDim.x >> 6) + wave; tile < n_tiles; tile += stride) {
        const long long row = tile * 32 + j;
        const bool valid = row < M;
        vec8 cur[NK], fwd[NK];
        TL::load(cur, dLdy, row, h, valid);
        // derivative of the output activation, applied on the T tile (kernel_esimd.h:193-201)
        if (out_act != TNN_ACT_NONE) {
            TL::load(fwd, interm_fwd + (size_t)n_mats * mat, row, h, valid);
#pragma unroll
            for (int kb = 0; kb < NK; ++kb) {
                f32x8 v;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float g = (float)cur[kb][e], f = (float)fwd[kb][e];
                    v[e] = (out_act == TNN_ACT_RELU) ? ((f <= 0.0f) ? 0.0f : g) : as_fp32(g * (f * (1.0f - f)));
                }
                cur[kb] = __builtin_convertvector(v, vec8);
            }
        }
        if (interm_bwd) TL::store(cur, interm_bwd + (size_t)(n_mats - 1) * mat, row, h, valid);

        f32x16 acc[NI];
        for (int l = n_mats - 1; l > 0; --l) {
            // the forward activation of layer l-1 that gates delta_{l-1}; issued before the MFMAs
            if (act != TNN_ACT_NONE) TL::load(fwd, interm_fwd + (size_t)l * mat, row, h, valid);
            TL::template matmul<W_IN_LDS>(acc, cur, lds_w, wprep_bwd, l, lane);
            if (act == TNN_ACT_RELU)
                TL::template bwd_repack<TNN_ACT_RELU>(cur, acc, fwd);
            else if (act == TNN_ACT_SIGMOID)
                TL::template bwd_repack<TNN_ACT_SIGMOID>(cur, acc, fwd);
            else
                TL::template repack<TNN_ACT_NONE>(cur, acc);
            if (interm_bwd) TL::store(cur, interm_bwd + (size_t)(l - 1) * mat, row, h, valid);
        }
        if (dLdx) {
            TL::template matmul<W_IN_LDS>(acc, cur, lds_w, wprep_bwd, 0, lane);
            TL::template repack<TNN_ACT_NONE>(cur, acc);
            TL::store(cur, dLdx, row, h, valid);
        }
    }
}

// ------------------------------------------------------------------------------------------
// Weight gradients: dW_l[n][k] = sum_m delta_l[m][n] * a_l[m][k]   (kernel_esimd.h:230-239)
// ------------------------------------------------------------------------------------------
constexpr int kDwThreads = 256;
constexpr int kDwSlab = 64; // rows staged in LDS per step

// Contraction runs over batch rows, which the streaming kernels keep one-per-lane; both operands are
// therefore transposed through LDS: a slab of rows is stored row-major and read back column-wise.
// Workgroup (l, c) reduces rows [c*rows_per_chunk, (c+1)*rows_per_chunk) of matrix l into one (or, for
// W <= 32, four) fp32 partial W x W tiles in the workspace; train_reduce_kernel sums the partials.
template <typename T, int W>
__global__ void __launch_bounds__(kDwThreads)
    mlp_dw_partial_kernel(const T *__restrict__ interm_bwd, const T *__restrict__ interm_fwd, float *__restrict__ partials,
                          int n_mats, long long M, long long rows_per_chunk) {
    typedef typename Storage<T>::vec8 vec8;
    constexpr int NI = (W + 31) / 32;
    constexpr int PITCH = W + 8;                 // elements; keeps 16-byte alignment, skews banks
    constexpr int TILES = NI * NI;
    constexpr int TPW = (TILES + 3) / 4;         // tiles per wave (W=128: 4, W=64: 1, else 1)
    constexpr bool SPLIT_ROWS = (TILES == 1);    // W <= 32: waves split the rows of a slab instead
    __shared__ __attribute__((aligned(16))) T lds_d[kDwSlab * PITCH];
    __shared__ __attribute__((aligned(16))) T lds_a[kDwSlab * PITCH];

    const int l = blockIdx.y;
    const long long chunk = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 31, h = lane >> 5;
    const T *dmat = interm_bwd + (size_t)l * M * W;
    const T *amat = interm_fwd + (size_t)l * M * W;
    const long long row0 = chunk * rows_per_chunk;
    long long row_end = row0 + rows_per_chunk;
    if (row_end > M) row_end = M;

    f32x16 acc[TPW];
#pragma unroll
    for (int t = 0; t < TPW; ++t) acc[t] = f32x16{};

    constexpr int CHUNKS_PER_ROW = W / 8;
    for (long long slab = row0; slab < row_end; slab += kDwSlab) {
        __syncthreads();
        for (int c = threadIdx.x; c < kDwSlab * CHUNKS_PER_ROW; c += kDwThreads) {
            const int r = c / CHUNKS_PER_ROW, cc = c % CHUNKS_PER_ROW;
            const long long row = slab + r;
            vec8 dv = vec8{}, av = vec8{};
            if (row < row_end) {
                dv = reinterpret_cast<const vec8 *>(dmat + row * W)[cc];
                av = reinterpret_cast<const vec8 *>(amat + row * W)[cc];
            }
            *reinterpret_cast<vec8 *>(&lds_d[r * PITCH + cc * 8]) = dv;
            *reinterpret_cast<vec8 *>(&lds_a[r * PITCH + cc * 8]) = av;
        }
        __syncthreads();
#pragma unroll
        for (int kb = 0; kb < kDwSlab / 16; ++kb) {
            if (SPLIT_ROWS && kb != wave) continue;
            const int rbase = 16 * kb + 8 * h;
            if (SPLIT_ROWS) {
                vec8 A = vec8{}, B = vec8{};
                if (i < W) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        A[t] = lds_d[(rbase + t) * PITCH + i];
                        B[t] = lds_a[(rbase + t) * PITCH + i];
                    }
                }
                acc[0] = Storage<T>::mfma(A, B, acc[0]);
            } else {
                // wave owns tiles (a, b): W=64 -> a = wave/2, b = wave%2 ; W=128 -> a = wave, b = 0..3
                const int a = (NI == 2) ? (wave >> 1) : wave;
                vec8 A;
#pragma unroll
                for (int t = 0; t < 8; ++t) A[t] = lds_d[(rbase + t) * PITCH + 32 * a + i];
#pragma unroll
                for (int tt = 0; tt < TPW; ++tt) {
                    const int b = (NI == 2) ? (wave & 1) : tt;
                    vec8 B;
#pragma unroll
                    for (int t = 0; t < 8; ++t) B[t] = lds_a[(rbase + t) * PITCH + 32 * b + i];
                    acc[tt] = Storage<T>::mfma(A, B, acc[tt]);
                }
            }
        }
    }
    // accumulator register r of lane (j = i, h) is element (row 8*(r/4) + 4*h + r%4, column j) of the tile
    const int ppw = SPLIT_ROWS ? 4 : 1;
    float *out = partials + (((size_t)chunk * ppw + (SPLIT_ROWS ? wave : 0)) * n_mats + l) * W * W;
#pragma unroll
    for (int tt = 0; tt < TPW; ++tt) {
        const int a = SPLIT_ROWS ? 0 : ((NI == 2) ? (wave >> 1) : wave);
        const int b = SPLIT_ROWS ? 0 : ((NI == 2) ? (wave & 1) : tt);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int n = 32 * a + 8 * (r >> 2) + 4 * h + (r & 3);
            const int k = 32 * b + i;
            if (n < W && k < W) out[n * W + k] = acc[tt][r];
        }
    }
}

// ------------------------------------------------------------------------------------------
// Host side
// ------------------------------------------------------------------------------------------
const DeviceInfo &device_info() {
    static thread_local DeviceInfo info[16];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) {
        static DeviceInfo bad;
        return bad;
    }
    if (!info[dev].ok) {
        hipDeviceProp_t p;
        if (hipGetDeviceProperties(&p, dev) == hipSuccess) {
            info[dev].n_cu = p.multiProcessorCount;
            info[dev].max_lds = p.maxSharedMemoryPerMultiProcessor ? p.maxSharedMemoryPerMultiProcessor : p.sharedMemPerBlock;
            info[dev].ok = true;
        }
    }
    return info[dev];
}

// LDS the weights may take and still leave room for two workgroups per CU.
constexpr size_t kLdsBudget = 144 * 1024;

// Grid of a streaming kernel: as many workgroups as the device holds at once (registers and LDS decide),
// capped by the number of 32-row tiles. The result per kernel is cached.
static long long stream_grid(const void *kernel, size_t lds_bytes, size_t M, int n_cu) {
    struct Entry {
        const void *k;
        size_t lds;
        int per_cu;
    };
    static thread_local Entry cache[64];
    static thread_local int n_cache = 0;
    int per_cu = 0;
    for (int i = 0; i < n_cache; ++i)
        if (cache[i].k == kernel && cache[i].lds == lds_bytes) per_cu = cache[i].per_cu;
    if (!per_cu) {
        int nb = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kernel, kFwdThreads, lds_bytes) != hipSuccess || nb < 1) {
            (void)hipGetLastError();
            nb = 1;
        }
        per_cu = nb;
        if (n_cache < 64) cache[n_cache++] = Entry{kernel, lds_bytes, per_cu};
    }
    const long long n_tiles = ((long long)M + 31) / 32;
    const int waves = kFwdThreads / 64;
    long long blocks = (n_tiles + waves - 1) / waves;
    if (blocks > (long long)n_cu * per_cu) blocks = (long long)n_cu * per_cu;
    return blocks < 1 ? 1 : blocks;
}

template <typename T, int W, int ACT, bool STORE_INTERM, int THREADS>
static int launch_forward_v(const tnn_mlp_desc *d, const void *wprep, const void *x, void *out, size_t M, hipStream_t s, int per_cu,
                            bool store_input = true) { // store_input = false: the width-128 streaming route may leave matrix 0 of `out` unwritten
    typedef typename Storage<T>::vec8 vec8;
    const int n_mats = d->n_hidden_layers + 1;
    const size_t wbytes = prepared_elems(d) * sizeof(T);
    const DeviceInfo &di = device_info();
    if (!di.ok) return fail(TNN_ERR_HIP, "no usable HIP device");
    const bool in_lds = wbytes <= kLdsBudget;
    if constexpr (W == 128) {
        // also for large batches when the weights would fit: the staging tiles of the whole-row stores do not fit beside
        // 128 KiB of weights, and the stores are what these passes are bound by (forward with stored activations, 4 matrices:
        // 442 -> 239 us at 2^20 rows, 124 -> 68 us at 2^18, no difference at 2^16, 1-3 us slower below; inference, 4 matrices:
        // 197 -> 182 us at 2^20 rows, 2 matrices: 143 -> 105 us)
        if (!in_lds || M >= 65536) { // stream the matrices through LDS, one layer at a time
            constexpr size_t lds = 2 * (size_t)Tile<T, W>::NI * Tile<T, W>::NK * kWaveSize * sizeof(vec8);
            constexpr long long round = (kStreamThreads / 64) * kStreamTiles * 32;
            long long g = ((long long)M + round - 1) / round;
            if (g > di.n_cu) g = di.n_cu;
            const bool fits32 = (unsigned long long)M * W * sizeof(T) <= Tile<T, W>::kMaxBufferBytes;
            const bool streaming = !STORE_INTERM || (unsigned long long)(n_mats + 1) * M * W * sizeof(T) > (256ull << 20);
            const size_t lds_staged = lds + (kStreamThreads / 64) * (size_t)Tile<T, W>::TILE_BYTES;
            auto k0 = mlp_forward_stream_kernel<T, W, ACT, STORE_INTERM, 0>;
            auto k1 = mlp_forward_stream_kernel<T, W, ACT, STORE_INTERM, 1>;
            auto k2 = mlp_forward_stream_kernel<T, W, ACT, STORE_INTERM, 2>;
            auto k = !fits32 ? k0 : (streaming ? k2 : k1);
            const size_t lds_k = fits32 ? lds_staged : lds;
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_k) != hipSuccess)
                return fail(TNN_ERR_HIP, "cannot reserve %zu bytes of LDS", lds_k);
            TNN_LAUNCH(k, dim3((unsigned)g), dim3(kStreamThreads), lds_k, s, (const vec8 *)wprep, (const T *)x, (T *)out, n_mats,
                       d->output_activation, (long long)M, store_input ? 1 : 0);
            return check_launch("mlp_forward_stream_kernel");
        }
    }
    const long long n_tiles = ((long long)M + 31) / 32;
    const int waves = THREADS / 64;
    long long blocks = (n_tiles + waves - 1) / waves;
    if (in_lds && wbytes * per_cu > 160 * 1024) per_cu = (int)(160 * 1024 / wbytes);
    if (blocks > (long long)di.n_cu * per_cu) blocks = (long long)di.n_cu * per_cu;
    if (blocks < 1) blocks = 1;
    // Rows leave through a staged tile per wave (whole lines per store instruction) when that costs no workgroup per CU
    // and the matrix fits 32-bit offsets; with the streaming hint for an inference result, and for activations whose
    // volume exceeds the 256 MB of cache in front of the HBM (below that the backward pass finds them there).
    const size_t staged_bytes = wbytes + (size_t)waves * Tile<T, W>::TILE_BYTES;
    const bool staged = W <= 64 && in_lds && staged_bytes * per_cu <= 160 * 1024 &&
                        (unsigned long long)M * W * sizeof(T) <= Tile<T, W>::kMaxBufferBytes;
    const bool streaming = !STORE_INTERM || (unsigned long long)(n_mats + 1) * M * W * sizeof(T) > (256ull << 20);
    if (staged) {
        auto k1 = mlp_forward_kernel<T, W, ACT, STORE_INTERM, true, THREADS, (W <= 64 ? 1 : 0)>;
        auto k2 = mlp_forward_kernel<T, W, ACT, STORE_INTERM, true, THREADS, (W <= 64 ? 2 : 0)>;
        auto k = streaming ? k2 : k1;
        // the reservation is a host round trip of several microseconds: once per kernel, device and size
        static thread_local size_t reserved[2][16] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return fail(TNN_ERR_HIP, "no usable HIP device");
        if (staged_bytes > 48 * 1024 && reserved[streaming][dev] < staged_bytes) {
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(k), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)staged_bytes) != hipSuccess)
                return fail(TNN_ERR_HIP, "cannot reserve %zu bytes of LDS", staged_bytes);
            reserved[streaming][dev] = staged_bytes;
        }
        TNN_LAUNCH(k, dim3((unsigned)blocks), dim3(THREADS), staged_bytes, s, (const vec8 *)wprep, (const T *)x,
                           (T *)out, n_mats, d->output_activation, (long long)M);
    } else if (in_lds) {
        auto k = mlp_forward_kernel<T, W, ACT, STORE_INTERM, true, THREADS>;
        if (wbytes > 48 * 1024 &&
            hipFuncSetAttribute(reinterpret_cast<const void *>(k), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)wbytes) != hipSuccess)
            return fail(TNN_ERR_HIP, "cannot reserve %zu bytes of LDS", wbytes);
        TNN_LAUNCH(k, dim3((unsigned)blocks), dim3(THREADS), wbytes, s, (const vec8 *)wprep, (const T *)x,
                           (T *)out, n_mats, d->output_activation, (long long)M);
    } else {
        auto k = mlp_forward_kernel<T, W, ACT, STORE_INTERM, false, THREADS>;
        TNN_LAUNCH(k, dim3((unsigned)blocks), dim3(THREADS), 0, s, (const vec8 *)wprep, (const T *)x, (T *)out,
                           n_mats, d->output_activation, (long long)M);
    }
    return check_launch("mlp_forward_kernel");
}

// 512 threads (8 waves, one 32-row tile each at a time) and two workgroups per CU: at most 128 VGPRs per lane,
// measured faster than 256-thread workgroups at higher counts and than variants that hold the next matrix's
// fragments in registers.
template <typename T, int W, int ACT, bool STORE_INTERM>
static int launch_forward_act(const tnn_mlp_desc *d, const void *wprep, const void *x, void *out, size_t M, hipStream_t s, bool store_input = true) {
    if constexpr (W <= 64) {
        // From two tiles per wave on a full chip: one workgroup of 16 waves per CU instead of two of 8, so that the weights
        // are staged once per CU (inference at 2^18 rows, w64 with 4 hidden layers: 13.7 -> 13.2 us); below that the
        // smaller workgroups spread over more CUs.
        const DeviceInfo &di = device_info();
        const size_t staged_bytes = prepared_elems(d) * sizeof(T) + 16 * (size_t)Tile<T, W>::TILE_BYTES;
        if (di.ok && (M + 31) / 32 >= (size_t)di.n_cu * 32 && staged_bytes <= 160 * 1024)
            return launch_forward_v<T, W, ACT, STORE_INTERM, 1024>(d, wprep, x, out, M, s, 1);
    }
    return launch_forward_v<T, W, ACT, STORE_INTERM, 512>(d, wprep, x, out, M, s, 2, store_input);
}

template <typename T, int W, bool STORE_INTERM>
static int launch_forward(const tnn_mlp_desc *d, const void *wprep, const void *x, void *out, size_t M, hipStream_t s, bool store_input = true) {
    switch (d->activation) {
    case TNN_ACT_RELU: return launch_forward_act<T, W, TNN_ACT_RELU, STORE_INTERM>(d, wprep, x, out, M, s, store_input);
    case TNN_ACT_SIGMOID: return launch_forward_act<T, W, TNN_ACT_SIGMOID, STORE_INTERM>(d, wprep, x, out, M, s, store_input);
    default: return launch_forward_act<T, W, TNN_ACT_NONE, STORE_INTERM>(d, wprep, x, out, M, s, store_input);
    }
}

// Delta propagation and (launch_dw) weight gradients as separate passes: widths up to 64 with more matrices than the
// kernel that forms both keeps on chip. Width 128 has launch_backward128.
template <typename T, int W>
static int launch_backward(const tnn_mlp_desc *d, const void *wprep_bwd, const void *dLdy, const void *interm_fwd,
                           void *interm_bwd, void *dLdx, size_t M, hipStream_t s) {
    typedef typename Storage<T>::vec8 vec8;
    const int n_mats = d->n_hidden_layers + 1;
    const size_t wbytes = prepared_elems(d) * sizeof(T);
    const DeviceInfo &di = device_info();
    if (!di.ok) return fail(TNN_ERR_HIP, "no usable HIP device");
    const bool in_lds = wbytes <= kLdsBudget;
    if (in_lds) {
        auto k = mlp_backward_kernel<T, W, true>;
        if (wbytes > 48 * 1024 &&
            hipFuncSetAttribute(reinterpret_cast<const void *>(k), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)wbytes) != hipSuccess)
            return fail(TNN_ERR_HIP, "cannot reserve %zu bytes of LDS", wbytes);
        const long long blocks = stream_grid(reinterpret_cast<const void *>(k), wbytes, M, di.n_cu);
        TNN_LAUNCH(k, dim3((unsigned)blocks), dim3(kFwdThreads), wbytes, s, (const vec8 *)wprep_bwd,
                           (const T *)dLdy, (const T *)interm_fwd, (T *)interm_bwd, (T *)dLdx, n_mats, d->activation,
                           d->output_activation, (long long)M);
    } else {
        const long long blocks = stream_grid(reinterpret_cast<const void *>(mlp_backward_kernel<T, W, false>), 0, M, di.n_cu);
        TNN_LAUNCH((mlp_backward_kernel<T, W, false>), dim3((unsigned)blocks), dim3(kFwdThreads), 0, s,
                           (const vec8 *)wprep_bwd, (const T *)dLdy, (const T *)interm_fwd, (T *)interm_bwd, (T *)dLdx,
                           n_mats, d->activation, d->output_activation, (long long)M);
    }
    return check_launch("mlp_backward_kernel");
}

struct DwPlan {
    long long rows_per_chunk;
    long long n_chunks;
    int partials_per_chunk;
    size_t partial_bytes; // fp32 partial tiles
    size_t delta_bytes;   // staging for the deltas when the caller does not want them
};

static DwPlan dw_plan(const tnn_mlp_desc *d, size_t M) {
    DwPlan p;
    const int W = d->width, n_mats = d->n_hidden_layers + 1;
    long long target_chunks = 256;
    long long rpc = ((long long)M + target_chunks - 1) / target_chunks;
    rpc = (rpc + kDwSlab - 1) / kDwSlab * kDwSlab;
    if (rpc < kDwSlab) rpc = kDwSlab;
    p.rows_per_chunk = rpc;
    p.n_chunks = M ? ((long long)M + rpc - 1) / rpc : 0;
    p.partials_per_chunk = (W <= 32) ? 4 : 1;
    p.partial_bytes = (size_t)p.n_chunks * p.partials_per_chunk * n_mats * W * W * sizeof(float);
    p.delta_bytes = (size_t)n_mats * M * W * 2;
    return p;
}

template <typename T, int W>
static int launch_dw(const tnn_mlp_desc *d, const void *interm_bwd, const void *interm_fwd, void *dW, int dW_is_fp32,
                     size_t M, float *partials, hipStream_t s) {
    const int n_mats = d->n_hidden_layers + 1;
    const DwPlan p = dw_plan(d, M);
    TNN_LAUNCH((mlp_dw_partial_kernel<T, W>), dim3((unsigned)p.n_chunks, (unsigned)n_mats), dim3(kDwThreads), 0, s,
                       (const T *)interm_bwd, (const T *)interm_fwd, partials, n_mats, (long long)M, p.rows_per_chunk);
    int rc = check_launch("mlp_dw_partial_kernel");
    if (rc) return rc;
    const int n_elems = n_mats * W * W;
    TNN_LAUNCH((train_reduce_kernel<T, false>), dim3(n_elems / 64), dim3(512), 0, s, partials, (const float *)nullptr,
               (int)(p.n_chunks * p.partials_per_chunk), n_elems, dW_is_fp32 ? (T *)nullptr : (T *)dW,
               dW_is_fp32 ? (float *)dW : (float *)nullptr, (float *)nullptr, AdamArgs{});
    return check_launch("train_reduce_kernel");
}

// Width 128: one launch per layer that forms delta_{l-1} and dW_l together (mlp_backward128.inc), then the reduction.
// With `targets` the top layer's launch forms dL/dy itself from the network's output (the last matrix of interm_fwd) and leaves
// the loss values as one sum per workgroup, which the reduction adds into *loss_sum; dLdy is then not read, and `tail` may ask
// for Adam on the reduced gradients inside the reduction (dW may then be null).
template <typename T>
static int launch_backward128(const tnn_mlp_desc *d, const void *wprep_bwd, const void *dLdy, const void *interm_fwd, void *deltas,
                              bool keep_top_delta, void *dW, int dW_is_fp32, void *dLdx, size_t M, float *partials, hipStream_t s,
                              const float *targets = nullptr, float loss_scale = 0.0f, float *loss_sum = nullptr, const void *x0 = nullptr,
                              const void *wprep_fwd = nullptr, // (with targets): the network's output is not in interm_fwd, the top launch forms it
                              const TrainTail &tail = TrainTail{}) {
    typedef typename Storage<T>::vec8 vec8;
    constexpr int W = 128;
    const int n_mats = d->n_hidden_layers + 1;
    const DwPlan p = dw_plan(d, M);
    const size_t mat = M * W, per_mat = (size_t)4 * 8 * 64;
    const bool reform = targets && wprep_fwd;
    auto k_top = reform ? mlp_layer_backward128_kernel<T, 3> : (targets ? mlp_layer_backward128_kernel<T, 2> : mlp_layer_backward128_kernel<T, 1>);
    auto k_mid = mlp_layer_backward128_kernel<T, 0>;
    auto k_pair = mlp_layer_pair_backward128_kernel<T>;
    const float inv_n = 1.0f / (float)(M * W);
    const size_t top_lds = reform ? LayerBwd128::pair_lds_bytes : LayerBwd128::lds_bytes;
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(k_top), hipFuncAttributeMaxDynamicSharedMemorySize, (int)top_lds) != hipSuccess)
        return fail(TNN_ERR_HIP, "cannot reserve %zu bytes of LDS", top_lds);
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(k_mid), hipFuncAttributeMaxDynamicSharedMemorySize, (int)LayerBwd128::lds_bytes) != hipSuccess)
        return fail(TNN_ERR_HIP, "cannot reserve %zu bytes of LDS", LayerBwd128::lds_bytes);
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(k_pair), hipFuncAttributeMaxDynamicSharedMemorySize, (int)LayerBwd128::pair_lds_bytes) != hipSuccess)
        return fail(TNN_ERR_HIP, "cannot reserve %zu bytes of LDS", LayerBwd128::pair_lds_bytes);
    const T *fwd = static_cast<const T *>(interm_fwd);
    const T *input0 = x0 ? static_cast<const T *>(x0) : fwd; // the first matrix's input: the caller's x, or its copy in front of the activations
    T *dl = static_cast<T *>(deltas);
    // from the loss nobody keeps the top layer's deltas: the workgroups' loss sums lie in that matrix's place
    float *loss_partials = (targets && loss_sum && !keep_top_delta && mat * sizeof(T) >= (size_t)p.n_chunks * sizeof(float))
                               ? reinterpret_cast<float *>(dl + (size_t)(n_mats - 1) * mat) : (float *)nullptr;
    if (targets && loss_sum && !loss_partials) return fail(TNN_ERR_INVALID_ARGUMENT, "no room for the loss sums of %lld workgroups", p.n_chunks);
    const vec8 *wb = static_cast<const vec8 *>(wprep_bwd);
    // the top layer by itself (it turns dL/dy or the loss into deltas first), then the layers below it two per launch, and
    // the first matrix by itself when their number is odd
    int l = n_mats - 1;
    while (l >= 0) {
        const bool top = (l == n_mats - 1);
        if (!top && l >= 1) {
            T *delta_out = l > 1 ? dl + (size_t)(l - 2) * mat : static_cast<T *>(dLdx);
            TNN_LAUNCH(k_pair, dim3((unsigned)p.n_chunks), dim3(kLayerBwdThreads), LayerBwd128::pair_lds_bytes, s, wb + (size_t)l * per_mat,
                       wb + (size_t)(l - 1) * per_mat, dl + (size_t)l * mat, fwd + (size_t)l * mat, l > 1 ? fwd + (size_t)(l - 1) * mat : input0,
                       keep_top_delta ? dl + (size_t)(l - 1) * mat : (T *)nullptr, delta_out, partials, n_mats, l, d->activation,
                       l > 1 ? d->activation : TNN_ACT_NONE, (long long)M, p.rows_per_chunk);
            const int rc = check_launch("mlp_layer_pair_backward128_kernel");
            if (rc) return rc;
            l -= 2;
            continue;
        }
        const T *delta_in = top ? static_cast<const T *>(dLdy) : dl + (size_t)l * mat;
        T *delta_out = l > 0 ? dl + (size_t)(l - 1) * mat : static_cast<T *>(dLdx);
        const int gate = l > 0 ? d->activation : TNN_ACT_NONE;
        TNN_LAUNCH((top ? k_top : k_mid), dim3((unsigned)p.n_chunks), dim3(kLayerBwdThreads), top ? top_lds : LayerBwd128::lds_bytes, s,
                   wb + (size_t)l * per_mat, delta_in, l > 0 ? fwd + (size_t)l * mat : input0, fwd + (size_t)n_mats * mat,
                   (top && keep_top_delta) ? dl + (size_t)l * mat : (T *)nullptr, delta_out, partials, n_mats, l, gate, d->output_activation, (long long)M,
                   p.rows_per_chunk, targets, loss_scale, inv_n, loss_partials,
                   (top && reform) ? static_cast<const vec8 *>(wprep_fwd) + (size_t)l * per_mat : (const vec8 *)nullptr);
        const int rc = check_launch("mlp_layer_backward128_kernel");
        if (rc) return rc;
        l -= 1;
    }
    if (tail.main_done && hipEventRecord(tail.main_done, s) != hipSuccess) return fail(TNN_ERR_HIP, "hipEventRecord failed");
    const int n_elems = n_mats * W * W;
    T *dW_T = (dW && !dW_is_fp32) ? (T *)dW : (T *)nullptr;
    float *dW_f32 = (dW && dW_is_fp32) ? (float *)dW : (float *)nullptr;
    if (tail.use_adam)
        TNN_LAUNCH((train_reduce_kernel<T, true>), dim3(n_elems / 64), dim3(512), 0, s, partials, loss_partials, (int)p.n_chunks, n_elems, dW_T, dW_f32,
                   loss_partials ? loss_sum : (float *)nullptr, tail.adam);
    else
        TNN_LAUNCH((train_reduce_kernel<T, false>), dim3(n_elems / 64), dim3(512), 0, s, partials, loss_partials, (int)p.n_chunks, n_elems, dW_T, dW_f32,
                   loss_partials ? loss_sum : (float *)nullptr, tail.adam);
    return check_launch("train_reduce_kernel");
}

// For tnn_mlp_train_step_l2 on width 128. The forward pass with stored activations that does not copy the input in front of
// them where its kernel can leave that out (2^20 rows: 268 MB less to write), ...
// without_output: the last layer is left out (the backward pass's top launch forms the network's output again from the last
// hidden layer, which lies where it always does); needs at least two hidden layers.
int forward128_for_training(const tnn_mlp_desc *desc, const void *wprep, const void *x, void *interm_fwd, size_t M, hipStream_t s, bool without_output) {
    tnn_mlp_desc d = *desc;
    if (without_output) {
        d.n_hidden_layers -= 1;
        d.output_activation = d.activation; // the last matrix that runs is a hidden layer's
    }
    if (desc->dtype == TNN_BF16) return launch_forward<bf16_t, 128, true>(&d, wprep, x, interm_fwd, M, s, false);
    return launch_forward<fp16_t, 128, true>(&d, wprep, x, interm_fwd, M, s, false);
}

// ... and loss and backward pass over those activations, the loss folded into the top layer's launch and the first matrix's
// input read from `x`. Workspace as tnn_mlp_backward's.
// wprep_fwd_if_no_output: the operand-order weights of the forward pass when interm_fwd holds no network output (see above), else null.
int backward128_from_loss(const tnn_mlp_desc *desc, const void *wprep_bwd, const void *x, const void *interm_fwd, const float *targets, float loss_scale,
                          float *loss_sum, void *dW, int dW_is_fp32, void *dLdx, size_t M, void *workspace, size_t workspace_bytes, hipStream_t s,
                          const void *wprep_fwd_if_no_output, const TrainTail &tail) {
    const DwPlan p = dw_plan(desc, M);
    const size_t partial_rounded = (p.partial_bytes + 255) & ~(size_t)255;
    const size_t need = partial_rounded + p.delta_bytes + 512;
    if (!workspace || workspace_bytes < need) return fail(TNN_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    uintptr_t base = (reinterpret_cast<uintptr_t>(workspace) + 255) & ~(uintptr_t)255;
    float *partials = reinterpret_cast<float *>(base);
    void *deltas = reinterpret_cast<void *>(base + partial_rounded);
    if (desc->dtype == TNN_BF16)
        return launch_backward128<bf16_t>(desc, wprep_bwd, nullptr, interm_fwd, deltas, false, dW, dW_is_fp32, dLdx, M, partials, s, targets, loss_scale,
                                          loss_sum, x, wprep_fwd_if_no_output, tail);
    return launch_backward128<fp16_t>(desc, wprep_bwd, nullptr, interm_fwd, deltas, false, dW, dW_is_fp32, dLdx, M, partials, s, targets, loss_scale,
                                      loss_sum, x, wprep_fwd_if_no_output, tail);
}

#define TNN_DISPATCH_TW(desc, CALL)                                                          \
    do {                                                                                     \
        if ((desc)->dtype == TNN_BF16) {                                                     \
            switch ((desc)->width) {                                                         \
            case 16: { typedef bf16_t T_; constexpr int W_ = 16; CALL; } break;              \
            case 32: { typedef bf16_t T_; constexpr int W_ = 32; CALL; } break;              \
            case 64: { typedef bf16_t T_; constexpr int W_ = 64; CALL; } break;              \
            default: { typedef bf16_t T_; constexpr int W_ = 128; CALL; } break;             \
            }                                                                                \
        } else {                                                                             \
            switch ((desc)->width) {                                                         \
            case 16: { typedef fp16_t T_; constexpr int W_ = 16; CALL; } break;              \
            case 32: { typedef fp16_t T_; constexpr int W_ = 32; CALL; } break;              \
            case 64: { typedef fp16_t T_; constexpr int W_ = 64; CALL; } break;              \
            default: { typedef fp16_t T_; constexpr int W_ = 128; CALL; } break;             \
            }                                                                                \
        }                                                                                    \
    } while (0)

// the widths below 128 (check_mlp_desc has let nothing else through)
#define TNN_DISPATCH_TW_UP_TO_64(desc, CALL)                                                 \
    do {                                                                                     \
        if ((desc)->dtype == TNN_BF16) {                                                     \
            switch ((desc)->width) {                                                         \
            case 16: { typedef bf16_t T_; constexpr int W_ = 16; CALL; } break;              \
            case 32: { typedef bf16_t T_; constexpr int W_ = 32; CALL; } break;              \
            default: { typedef bf16_t T_; constexpr int W_ = 64; CALL; } break;              \
            }                                                                                \
        } else {                                                                             \
            switch ((desc)->width) {                                                         \
            case 16: { typedef fp16_t T_; constexpr int W_ = 16; CALL; } break;              \
            case 32: { typedef fp16_t T_; constexpr int W_ = 32; CALL; } break;              \
            default: { typedef fp16_t T_; constexpr int W_ = 64; CALL; } break;              \
            }                                                                                \
        }                                                                                    \
    } while (0)

static int check_batch(size_t M) {
    // include/network/SwiftNetMLP.h:293-300: the batch must be a multiple of 8
    if (M == 0 || (M % 8) != 0) return fail(TNN_ERR_INVALID_ARGUMENT, "batch size %zu is not a positive multiple of 8", M);
    return TNN_OK;
}

// Everything Network::set_weights_matrices derives from packed parameters, in one pass: the packed copy in T with the
// weights that only see padding zeroed, its packed transpose, and both operand-order copies. A thread takes one slot of the
// operand-order index space (which covers every matrix element once, plus the empty half-tile at width 16).
template <typename T, typename SRC>
__global__ void set_packed_weights_kernel(const SRC *__restrict__ src, T *__restrict__ packed, T *__restrict__ packed_t, T *__restrict__ fwd,
                                          T *__restrict__ bwd, int W, int n_mats, int live_in, int live_out) {
    const int NI = (W + 31) / 32, NK = W / 16;
    const int per_mat = NI * NK * 512;
    const int total = n_mats * per_mat;
    for (int idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        const int l = idx / per_mat;
        int r = idx % per_mat;
        const int t = r & 7;
        const int lane = (r >> 3) & 63;
        r >>= 9;
        const int kb = r % NK, a = r / NK;
        const int h = lane >> 5, i = lane & 31;
        const int outer = 32 * a + swap23(i), inner = 16 * kb + 8 * h + t;
        T vf = (T)0.0f, vb = (T)0.0f;
        if (outer < W) {
            const size_t m = (size_t)l * W * W;
            // rows of the first matrix from live_in on and columns of the last matrix from live_out on only see padding
            auto weight = [&](int k, int n) { return ((l == 0 && k >= live_in) || (l == n_mats - 1 && n >= live_out)) ? (T)0.0f : (T)(float)src[m + packed_coord(k, n, W)]; };
            vf = weight(inner, outer);
            vb = weight(outer, inner);
            packed[m + packed_coord(inner, outer, W)] = vf;
            packed_t[m + packed_coord(outer, inner, W)] = vf; // element (k, n) of W is element (n, k) of its transpose
        }
        fwd[idx] = vf;
        bwd[idx] = vb;
    }
}

} // namespace tnn

using namespace tnn;

TNN_API int tnn_mlp_set_packed_weights(const tnn_mlp_desc *desc, const void *d_src_packed, int src_dtype, int unpadded_input_width,
                                       int unpadded_output_width, int use_bias, void *d_packed_T, void *d_packed_transposed_T,
                                       void *d_prepared_fwd, void *d_prepared_bwd, tnn_stream_t stream) {
    int rc = check_mlp_desc(desc);
    if (rc) return rc;
    if (!d_src_packed || !d_packed_T || !d_packed_transposed_T || !d_prepared_fwd || !d_prepared_bwd)
        return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    if (d_src_packed == d_packed_T || d_src_packed == d_packed_transposed_T) return fail(TNN_ERR_INVALID_ARGUMENT, "the source must not be one of the destinations");
    const int W = desc->width;
    if (unpadded_input_width > W || unpadded_output_width > W || unpadded_input_width <= 0 || unpadded_output_width <= 0)
        return fail(TNN_ERR_INVALID_ARGUMENT, "Padded weights width cannot be less than the unpadded.");
    // include/network/Network.h:191-202: with the bias trick the ones reach up to the next multiple of 16, and an input width
    // that already is one leaves the whole padded width live
    const int live_in = !use_bias ? unpadded_input_width : (unpadded_input_width % 16 == 0 ? W : (unpadded_input_width / 16 + 1) * 16);
    if (live_in > W) return fail(TNN_ERR_INVALID_ARGUMENT, "one_padded_input_width > padded_input_width, the input width is too small.");
    const int n_mats = desc->n_hidden_layers + 1;
    const int total = (int)prepared_elems(desc);
    const int blocks = (total + 255) / 256;
    hipStream_t s = as_stream(stream);
#define TNN_SPW(T_, S_)                                                                                                                          \
    TNN_LAUNCH((set_packed_weights_kernel<T_, S_>), dim3(blocks), dim3(256), 0, s, (const S_ *)d_src_packed, (T_ *)d_packed_T, (T_ *)d_packed_transposed_T, \
               (T_ *)d_prepared_fwd, (T_ *)d_prepared_bwd, W, n_mats, live_in, unpadded_output_width)
    if (desc->dtype == TNN_BF16) {
        if (src_dtype == TNN_FP32) TNN_SPW(bf16_t, float);
        else if (src_dtype == TNN_BF16) TNN_SPW(bf16_t, bf16_t);
        else if (src_dtype == TNN_FP16) TNN_SPW(bf16_t, fp16_t);
        else return fail(TNN_ERR_UNSUPPORTED, "src_dtype %d", src_dtype);
    } else {
        if (src_dtype == TNN_FP32) TNN_SPW(fp16_t, float);
        else if (src_dtype == TNN_BF16) TNN_SPW(fp16_t, bf16_t);
        else if (src_dtype == TNN_FP16) TNN_SPW(fp16_t, fp16_t);
        else return fail(TNN_ERR_UNSUPPORTED, "src_dtype %d", src_dtype);
    }
#undef TNN_SPW
    return check_launch("set_packed_weights_kernel");
}

TNN_API size_t tnn_mlp_prepared_bytes(const tnn_mlp_desc *desc) {
    if (check_mlp_desc(desc)) return 0;
    return prepared_elems(desc) * 2;
}

TNN_API int tnn_mlp_prepare_weights(const tnn_mlp_desc *desc, const void *d_packed, int src_is_fp32, void *d_prepared_fwd,
                                    void *d_prepared_bwd, tnn_stream_t stream) {
    int rc = check_mlp_desc(desc);
    if (rc) return rc;
    if (!d_packed) return fail(TNN_ERR_INVALID_ARGUMENT, "d_packed is NULL");
    const int n_mats = desc->n_hidden_layers + 1;
    const int total = (int)prepared_elems(desc);
    const int blocks = (total + 255) / 256;
    hipStream_t s = as_stream(stream);
    if (desc->dtype == TNN_BF16) {
        if (src_is_fp32)
            TNN_LAUNCH((prepare_weights_kernel<bf16_t, float>), dim3(blocks), dim3(256), 0, s, (const float *)d_packed,
                               (bf16_t *)d_prepared_fwd, (bf16_t *)d_prepared_bwd, desc->width, n_mats);
        else
            TNN_LAUNCH((prepare_weights_kernel<bf16_t, bf16_t>), dim3(blocks), dim3(256), 0, s,
                               (const bf16_t *)d_packed, (bf16_t *)d_prepared_fwd, (bf16_t *)d_prepared_bwd, desc->width,
                               n_mats);
    } else {
        if (src_is_fp32)
            TNN_LAUNCH((prepare_weights_kernel<fp16_t, float>), dim3(blocks), dim3(256), 0, s, (const float *)d_packed,
                               (fp16_t *)d_prepared_fwd, (fp16_t *)d_prepared_bwd, desc->width, n_mats);
        else
            TNN_LAUNCH((prepare_weights_kernel<fp16_t, fp16_t>), dim3(blocks), dim3(256), 0, s,
                               (const fp16_t *)d_packed, (fp16_t *)d_prepared_fwd, (fp16_t *)d_prepared_bwd, desc->width,
                               n_mats);
    }
    return check_launch("prepare_weights_kernel");
}

TNN_API int tnn_mlp_inference(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_x, void *d_y, size_t M,
                              tnn_stream_t stream) {
    int rc = check_mlp_desc(desc);
    if (rc) return rc;
    if ((rc = check_batch(M))) return rc;
    if (!d_prepared_fwd || !d_x || !d_y) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    TNN_DISPATCH_TW(desc, rc = (launch_forward<T_, W_, false>(desc, d_prepared_fwd, d_x, d_y, M, as_stream(stream))));
    return rc;
}

TNN_API int tnn_mlp_forward(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_x, void *d_interm_fwd,
                            size_t M, tnn_stream_t stream) {
    int rc = check_mlp_desc(desc);
    if (rc) return rc;
    if ((rc = check_batch(M))) return rc;
    if (!d_prepared_fwd || !d_x || !d_interm_fwd) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    TNN_DISPATCH_TW(desc, rc = (launch_forward<T_, W_, true>(desc, d_prepared_fwd, d_x, d_interm_fwd, M, as_stream(stream))));
    return rc;
}

TNN_API size_t tnn_mlp_backward_workspace_bytes(const tnn_mlp_desc *desc, size_t M) {
    if (check_mlp_desc(desc)) return 0;
    const DwPlan p = dw_plan(desc, M);
    return ((p.partial_bytes + 255) & ~(size_t)255) + p.delta_bytes + 512;
}

TNN_API int tnn_mlp_backward(const tnn_mlp_desc *desc, const void *d_prepared_bwd, const void *d_dLdy,
                             const void *d_interm_fwd, void *d_interm_bwd, void *d_dW, int dW_is_fp32, void *d_dLdx,
                             size_t M, void *d_workspace, size_t workspace_bytes, tnn_stream_t stream) {
    int rc = check_mlp_desc(desc);
    if (rc) return rc;
    if ((rc = check_batch(M))) return rc;
    if (!d_prepared_bwd || !d_dLdy || !d_interm_fwd || !d_dW) return fail(TNN_ERR_INVALID_ARGUMENT, "NULL pointer argument");
    const DwPlan p = dw_plan(desc, M);
    const size_t partial_rounded = (p.partial_bytes + 255) & ~(size_t)255;
    const size_t need = partial_rounded + (d_interm_bwd ? 0 : p.delta_bytes) + 512;
    if (!d_workspace || workspace_bytes < need)
        return fail(TNN_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    // 256-byte aligned partial tiles first, delta staging after them
    uintptr_t base = (reinterpret_cast<uintptr_t>(d_workspace) + 255) & ~(uintptr_t)255;
    float *partials = reinterpret_cast<float *>(base);
    void *deltas = d_interm_bwd ? d_interm_bwd : reinterpret_cast<void *>(base + partial_rounded);
    hipStream_t s = as_stream(stream);
    // one kernel for deltas and weight gradients where the shape has it (width <= 64, up to 9 matrices); the deltas are
    // then written only if the caller asked for them
    rc = fused_backward(desc, d_prepared_bwd, d_dLdy, d_interm_fwd, d_interm_bwd, d_dW, dW_is_fp32, d_dLdx, M, partials, p.partial_bytes, s);
    if (rc != TNN_ERR_UNSUPPORTED) return rc;
    if (desc->width == 128) {
        if (desc->dtype == TNN_BF16)
            return launch_backward128<bf16_t>(desc, d_prepared_bwd, d_dLdy, d_interm_fwd, deltas, d_interm_bwd != nullptr, d_dW, dW_is_fp32, d_dLdx, M,
                                              partials, s);
        return launch_backward128<fp16_t>(desc, d_prepared_bwd, d_dLdy, d_interm_fwd, deltas, d_interm_bwd != nullptr, d_dW, dW_is_fp32, d_dLdx, M,
                                          partials, s);
    }
    TNN_DISPATCH_TW_UP_TO_64(desc, rc = (launch_backward<T_, W_>(desc, d_prepared_bwd, d_dLdy, d_interm_fwd, deltas, d_dLdx, M, s)));
    if (rc) return rc;
    TNN_DISPATCH_TW_UP_TO_64(desc, rc = (launch_dw<T_, W_>(desc, deltas, d_interm_fwd, d_dW, dW_is_fp32, M, partials, s)));
    return rc;
}
